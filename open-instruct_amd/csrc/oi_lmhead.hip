// Fused lm_head projection + per-token logprob / entropy for gfx950, logits never materialised.
//
// One bf16 MFMA main loop, C[m, n] = sum_k a(m, k) * b(n, k), serves four kernels that differ in
// what they do with the fp32 tile and in the memory order of their operands (k-contiguous: the k
// values of a row lie together; k-major: the rows of a k value lie together):
//
//   forward   a = W [V, H],  b = hidden [N, H]   both k-contiguous -> online (max, sum-exp,
//             sum exp*z) per token, merged over the vocabulary tiles of a work item
//   dz        a = W,         b = hidden          -> dZ = g * (onehot - softmax), bf16 [N, Vc]
//   d_hidden  a = dZ [N, Vc] k-contiguous, b = W [Vc, H] k-major -> fp32 accumulate over chunks
//   d_weight  a = dZ [N, Vc] k-major,      b = hidden [N, H] k-major -> bf16 rows of dW
//
// so the backward reads W, hidden and dZ where they lie: no transposed copies.
//
// Tile: 256 x 256 x 64 per 512-thread workgroup, 8 waves as 4 (m) x 2 (n), each wave 64 x 128 =
// 2 x 4 MFMA 32x32x16 accumulators.  With vocabulary as the m dim a lane's 16 accumulator
// registers of one MFMA tile belong to ONE token (column), so the softmax statistics reduce
// inside the lane.  LDS: a ring of five 32 KB operand slots (k-tiles of A and of B) filled by
// direct global->LDS loads of whole 128-byte line segments; the 16-byte chunks of a row are
// XOR-permuted so that fragment reads (16-byte reads of a k-contiguous image, transposing 8-byte
// reads of a k-major image) stay free of bank conflicts.  A launch is one resident workgroup per
// CU that draws tile ids from per-XCD counters.
#include "oi_common.h"

#include <type_traits>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int NTHREADS = 512;
constexpr int TILE_ELEMS = BM * BK;             // one operand tile in LDS, rows of 128 B, unpadded
constexpr int STAGE_STRIDE = 256 + 8;           // bf16 per row of the dZ staging tile
constexpr int LDS_ELEMS = 5 * TILE_ELEMS;       // 163840 B: the five-slot operand ring, all of a CU's LDS
static_assert(256 * STAGE_STRIDE <= LDS_ELEMS, "the dZ staging tile must fit");

typedef f32x16 AccTile[2][4];

// XCD-aware tile order.  Consecutive workgroup ids go round-robin to the 8 XCDs, each with its own
// L2; the 32 workgroups resident on one XCD form an 8 (m) x 4 (n) super-tile so that they share
// operand slabs in that L2.  The 8 XCDs take super-tiles that are neighbours along n and the sweep
// over n completes before m advances: the chip as a whole then works on one slab of A (the larger
// operand: lm_head rows, dZ rows) at a time, which stays in the memory-side cache while every n
// tile passes over it, instead of streaming all of A from HBM once per n super-tile.  Measured:
// +4 to +7 % on every shape of the lm_head path (the kernel runs at the chip's power limit, and
// HBM traffic costs power).
__device__ __forceinline__ bool tile_of_pid(int64_t pid, int64_t tiles_m, int64_t tiles_n, int64_t* tm, int64_t* tn) {
    const int64_t xcd = pid & 7, local = pid >> 3;
    const int64_t nsn = (tiles_n + 3) / 4;
    const int64_t st = (local >> 5) * 8 + xcd, inner = local & 31;
    *tm = (st / nsn) * 8 + (inner & 7);
    *tn = (st % nsn) * 4 + (inner >> 3);
    return *tm < tiles_m && *tn < tiles_n;
}
// number of ids to enumerate (whole super-tiles, a multiple of 256)
__host__ __device__ inline int64_t pids_for_tiles(int64_t tiles_m, int64_t tiles_n) {
    const int64_t nst = ((tiles_m + 7) / 8) * ((tiles_n + 3) / 4);
    return ((nst + 7) / 8) * 8 * 32;
}

// Work queue.  A launch of the tile kernels is one workgroup per CU (the LDS ring leaves room for
// no second one) that stays for the whole launch and draws tile ids from a counter, rather than
// one short-lived workgroup per tile.  There is one counter per XCD (workgroup b is taken to run
// on XCD b mod 8, as the tile order assumes), so the ids an XCD draws are the ones tile_of_pid
// maps onto shared operand slabs; a wrong guess costs cache hits, never correctness.  The XCDs do
// not finish their shares together (measured on the forward: 1.7 ms apart in an 18 ms launch), so
// a workgroup whose own queue has run dry goes on with the queues of the other XCDs, one after the
// other: the launch then ends within one work item for all of them.  The next id is requested
// before the current tile is computed and handed to the other waves through one LDS word
// afterwards.  `counters` are 8 zeroed words; every workgroup leaves each of them raised past the
// number of ids at most once.
constexpr int QUEUE_WORDS = 8;
constexpr int FWD_QUEUE_WORDS = 2 * QUEUE_WORDS;  // the forward hands out its long and its short items from two sets of queues
// threadIdx.x as a value the optimiser cannot trace: everything derived from it (fragment and
// epilogue addresses) is then recomputed per tile instead of being hoisted out of the tile loop,
// where it would stay live through the main loop and push accumulators into scratch
__device__ __forceinline__ int opaque_tid() {
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}
template <class Body>
__device__ __forceinline__ void for_each_tile(uint32_t* __restrict__ counters, int64_t tiles_m, int64_t tiles_n,
                                              uint16_t* lds, Body&& body) {
    const uint32_t xcd = blockIdx.x & 7;
    const uint32_t locals = (uint32_t)(pids_for_tiles(tiles_m, tiles_n) >> 3);  // ids per queue
    // the word sits in the fifth ring slot, which the main loop first writes after its first barrier
    volatile uint32_t* mailbox = reinterpret_cast<volatile uint32_t*>(lds + 4 * BM * BK);
    constexpr uint32_t NONE = 0xffffffffu;
    // thread 0 only: the queues of XCDs xcd .. xcd + dry - 1 (mod 8) are known to be empty and
    // `drawn` came from the queue of XCD xcd + dry
    uint32_t dry = 0, drawn = 0;
    // a kernel may run several of these loops back to back over the same word: every wave must have
    // read the previous loop's last value before thread 0 writes this loop's first one
    __syncthreads();
    auto resolve = [&]() -> uint32_t {
        for (;;) {
            if (drawn < locals) return drawn * 8 + ((xcd + dry) & 7);
            if (++dry == 8) return NONE;
            drawn = atomicAdd(&counters[(xcd + dry) & 7], 1u);
        }
    };
    if (threadIdx.x == 0) {
        drawn = atomicAdd(&counters[xcd], 1u);
        *mailbox = resolve();
    }
    __syncthreads();
    uint32_t pid = __builtin_amdgcn_readfirstlane(*mailbox);
    while (pid != NONE) {
        // in flight while the tile is computed
        if (threadIdx.x == 0 && dry < 8) drawn = atomicAdd(&counters[(xcd + dry) & 7], 1u);
        int64_t tm, tn;
        if (tile_of_pid((int64_t)pid, tiles_m, tiles_n, &tm, &tn)) body(tm, tn);
        __syncthreads();  // the tile's last use of the LDS is over
        if (threadIdx.x == 0) *mailbox = dry < 8 ? resolve() : NONE;
        __syncthreads();
        pid = __builtin_amdgcn_readfirstlane(*mailbox);
    }
}
// fallback used by the stand-alone GEMM entry point, which has no workspace for a counter: one
// workgroup per tile id
__device__ __forceinline__ bool tile_of_block(int64_t tiles_m, int64_t tiles_n, int64_t* tm, int64_t* tn) {
    return tile_of_pid(blockIdx.x, tiles_m, tiles_n, tm, tn);
}
inline unsigned grid_for_tiles(int64_t tiles_m, int64_t tiles_n) { return (unsigned)pids_for_tiles(tiles_m, tiles_n); }

// LDS tile layout: row r of an operand tile holds its 64 k-values as eight 16-byte chunks; chunk c
// is stored at position c ^ swz(r).  With that permutation the 16-byte fragment reads of 16
// consecutive rows at one logical chunk fall on distinct banks, and the rows stay unpadded, which
// the direct global->LDS loads need (a wave's 64 lanes fill 1 KB of consecutive LDS).
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

#define OI_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define OI_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

// Wait until at most PENDING of this wave's global->LDS loads are still in flight, then meet the
// other waves.  A bare s_barrier (no fence) keeps the compiler from draining the loads that were
// issued for later k-tiles.
template <int PENDING>
__device__ __forceinline__ void wait_loads_and_barrier() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PENDING) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// acc = A[m0 : m0+256, :K] * B[n0 : n0+256, :K]^T.  Rows past M / N are clamped onto the last
// valid row (their results are discarded by the epilogues); K must be a multiple of 64.
//
// Operand tiles reach the LDS by direct global->LDS loads (no VGPR staging, no LDS store
// instructions).  Eight consecutive lanes fetch the eight 16-byte chunks of one 128-byte row
// segment, i.e. whole cache lines.  The path from L2 into the LDS delivers a 64 KB k-tile to a CU
// in about the time the matrix pipe needs to multiply it, so the loads must be in flight all the
// time: issued in one burst per k-tile they back up in the load unit and hold the issuing waves
// (and their MFMAs) for twice the MFMA time of that k-step.  Spreading them needs a free
// destination throughout the k-tile, which two full stages cannot give (the stage being read is
// the only candidate), hence a ring of FIVE operand slots of 32 KB, all of a CU's 160 KB:
// k-tile t reads A_t and B_t from two slots, A_(t+1) and B_(t+1) are landing in two more,
// A_(t+2) goes into the fifth at any time, and B_(t+2) takes A_t's slot once the barrier near the
// end of k-tile t has passed.
// Wave w owns rows [32 w, 32 w + 32) of both operand tiles: 4 + 4 loads of 1 KB per k-tile.
constexpr int NSLOT = 5;
constexpr int64_t MAX_LD = (int64_t)1 << 22;  // 255 rows * ld * 2 bytes must fit 32 bits
__device__ __forceinline__ int ring_slot(int s) { return s >= NSLOT ? s - NSLOT : s; }

// One operand of a tile product, in either of two memory layouts.
//   k-contiguous (KM = false): element (row, k) at p[row * ld + k]; the tile takes rows
//     [r0, r0 + 256), rows at or past `extent` are clamped onto the last valid one.
//   k-major (KM = true): element (row, k) at p[k * ld + row]; the tile takes columns
//     [r0, r0 + 256) of every k row, 16-byte column chunks past `extent` (a multiple of 8) are
//     clamped onto the last valid chunk, k rows at or past `k_valid` onto the last valid row (the
//     other operand must hold zeros there).  This is the layout in which a matrix is its own
//     transpose operand: W [V, H] as the B operand of dZ * W, hidden [N, H] and dZ [N, V] as the
//     operands of dZ^T * hidden, with no transposed copies in memory.
// In both cases the results of clamped rows / columns are garbage that the epilogues discard.
struct Operand {
    const uint16_t* p;
    int64_t ld, r0, extent, k_valid;
};

typedef short v4i16 __attribute__((ext_vector_type(4)));

// acc = A_tile * B_tile^T over k in [0, K), K a multiple of 64.
//
// Operand tiles reach the LDS by direct global->LDS loads (no VGPR staging, no LDS store
// instructions), whole 128-byte cache-line segments per 8 lanes.  The path from L2 into the LDS
// delivers a 64 KB k-tile to a CU in about the time the matrix pipe needs to multiply it, so the
// loads must be in flight all the time: issued in one burst per k-tile they back up in the load
// unit and hold the issuing waves (and their MFMAs) for twice the MFMA time of that k-step.
// Spreading them needs a free destination throughout the k-tile, which two full stages cannot give
// (the stage being read is the only candidate), hence a ring of FIVE operand slots of 32 KB, all
// of a CU's 160 KB: k-tile t reads A_t and B_t from two slots, A_(t+1) and B_(t+1) are landing in
// two more, A_(t+2) goes into the fifth at any time, and B_(t+2) takes A_t's slot once the barrier
// near the end of k-tile t has passed.  Every wave issues 4 + 4 loads of 1 KB per k-tile.
//
// LDS image of a k-contiguous operand tile: [256 rows][64 k], the eight 16-byte chunks of a row
// stored at c ^ swz(row); wave w loads rows [32 w, 32 w + 32); fragments are 16-byte reads.
// LDS image of a k-major operand tile: [64 k][256 columns], the 32 chunks of a k row stored at
// c ^ 4 (k & 3); wave w loads k rows [8 w, 8 w + 8); fragments come through the transposing read
// ds_read_b64_tr_b16: in a group of 16 lanes, lane s points at (k0 + s / 4, 4 columns from
// 4 (s % 4)) and lane i receives column i at k0 .. k0 + 3, which is the MFMA operand layout (row
// per lane, consecutive k per register).  The permutation puts the four k rows of such a read on
// different banks.
template <bool A_KM, bool B_KM>
__device__ __forceinline__ void gemm_tile(AccTile& acc, const Operand& A, const Operand& B, int64_t K, uint16_t* lds) {
    const int tid = opaque_tid();
    // the wave index as a scalar: the LDS destinations of the loads (M0) then take no VALU work
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 3, wn = wave >> 2;

#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int64_t ktiles = K / BK;
    // loader side.  Addresses are a uniform 64-bit base (tile origin + k offset) plus a 32-bit byte
    // offset per lane; for a k-major operand the lanes' offsets of the last k-tile differ (its k
    // rows may end early), `last` holds those.
    struct Loader {
        const char* tile;    // origin of the tile in global memory
        int64_t k_step;      // bytes from one k-tile to the next
        uint32_t off[4];     // per-lane byte offsets of the four loads
        uint32_t last[4];    // the same for the last k-tile
        int lds_block;       // elements between the LDS destinations of consecutive loads
        int lds_wave;        // element offset of this wave's first load inside a slot
    };
    auto make_loader = [&](const Operand& op, auto km_tag) {
        constexpr bool KM = decltype(km_tag)::value;
        Loader L;
        if constexpr (!KM) {
            L.tile = reinterpret_cast<const char*>(op.p + op.r0 * op.ld);
            L.k_step = BK * 2;
            const int last_row = (int)((op.extent - 1 - op.r0) < 255 ? (op.extent - 1 - op.r0) : 255);
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int r = wave * 32 + b * 8 + (lane >> 3);
                const int c = (lane & 7) ^ swz(r);
                L.off[b] = (uint32_t)(r < last_row ? r : last_row) * (uint32_t)(op.ld * 2) + c * 16;
                L.last[b] = L.off[b];
            }
            L.lds_block = 8 * BK;
            L.lds_wave = wave * 32 * BK;
        } else {
            L.tile = reinterpret_cast<const char*>(op.p);
            L.k_step = BK * op.ld * 2;
            const int last_k = (int)(op.k_valid - 1 - (ktiles - 1) * BK);  // inside the last k-tile
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int kk = wave * 8 + b * 2 + (lane >> 5);
                const int c = (lane & 31) ^ (4 * (kk & 3));
                int64_t col = op.r0 + c * 8;
                col = col + 8 <= op.extent ? col : op.extent - 8;
                L.off[b] = (uint32_t)kk * (uint32_t)(op.ld * 2) + (uint32_t)(col * 2);
                L.last[b] = (uint32_t)(kk < last_k ? kk : last_k) * (uint32_t)(op.ld * 2) + (uint32_t)(col * 2);
            }
            L.lds_block = 2 * 256;
            L.lds_wave = wave * 8 * 256;
        }
        return L;
    };
    const Loader la = make_loader(A, std::integral_constant<bool, A_KM>{});
    const Loader lb = make_loader(B, std::integral_constant<bool, B_KM>{});
    // k-tiles past the end are never requested by the loop below; the prologue may ask for k-tile 1
    // of a one-k-tile product and then re-reads k-tile 0 into a slot nobody reads
    auto k_src = [&](const Loader& L, int64_t kt) {
        const uint64_t v = reinterpret_cast<uint64_t>(L.tile + (kt < ktiles ? kt : ktiles - 1) * L.k_step);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
    };
    // one 1 KB load: block b of this wave's share of an operand k-tile into ring slot `slot`
    auto load_block = [&](const Loader& L, const char* src, uint32_t off, int slot, int b) {
        __builtin_amdgcn_global_load_lds(OI_GLOBAL_PTR(src + off),
                                         OI_LDS_PTR(lds + slot * TILE_ELEMS + L.lds_wave + b * L.lds_block), 16, 0, 0);
    };
    // ring slots: A_t -> (2 t) mod 5, B_t -> (2 t + 1) mod 5
    {
        const char* a_k0 = k_src(la, 0);
        const char* b_k0 = k_src(lb, 0);
        const char* a_k1 = k_src(la, 1);
        const char* b_k1 = k_src(lb, 1);
        const bool t0_last = ktiles == 1, t1_last = ktiles <= 2;
#pragma unroll
        for (int b = 0; b < 4; ++b) load_block(la, a_k0, t0_last ? la.last[b] : la.off[b], 0, b);
#pragma unroll
        for (int b = 0; b < 4; ++b) load_block(lb, b_k0, t0_last ? lb.last[b] : lb.off[b], 1, b);
#pragma unroll
        for (int b = 0; b < 4; ++b) load_block(la, a_k1, t1_last ? la.last[b] : la.off[b], 2, b);
#pragma unroll
        for (int b = 0; b < 3; ++b) load_block(lb, b_k1, t1_last ? lb.last[b] : lb.off[b], 3, b);
    }

    // consumer side: element offsets of this lane's fragments inside a slot
    const int lr = lane & 31, h = lane >> 5;
    // k-contiguous image: k-step ks flips the stored chunk by (2 ks); rows 32 apart share the
    // same permutation
    const int pg = h ^ swz(lr);
    const int a_base = (wm * 64 + lr) * BK + pg * 8, b_base = (wn * 128 + lr) * BK + pg * 8;
    // k-major image: source lane s of a 16-lane group points at k row (s >> 2) of the lane's
    // half-k-step and at 4 columns from 4 (s & 3) of the group's 16; one address per 32-row tile
    // because the column permutation reaches the bits that select the tile
    const int s16 = lane & 15, e4 = s16 >> 2, g16 = (lane >> 4) & 1;
    int a_km[2], b_km[4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
        a_km[i] = (h * 8 + e4) * 256 + (((wm * 8 + i * 4 + g16 * 2 + ((s16 & 3) >> 1)) ^ (4 * e4)) * 8) + 4 * (s16 & 1);
#pragma unroll
    for (int j = 0; j < 4; ++j)
        b_km[j] = (h * 8 + e4) * 256 + (((wn * 16 + j * 4 + g16 * 2 + ((s16 & 3) >> 1)) ^ (4 * e4)) * 8) + 4 * (s16 & 1);
    auto read_tr = [&](const uint16_t* p) {
        // rows k0 .. k0 + 3 and k0 + 4 .. k0 + 7 of the lane's half-k-step
        const v4i16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) v4i16*)OI_LDS_PTR(const_cast<uint16_t*>(p)));
        const v4i16 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) v4i16*)OI_LDS_PTR(const_cast<uint16_t*>(p + 4 * 256)));
        const short __attribute__((ext_vector_type(8))) both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, both);
    };
    auto read_a = [&](int slot, int ks, int i) {
        if constexpr (A_KM) return read_tr(lds + slot * TILE_ELEMS + ks * 16 * 256 + a_km[i]);
        else return *reinterpret_cast<const bf16x8*>(lds + slot * TILE_ELEMS + (a_base ^ (ks * 16)) + i * 32 * BK);
    };
    auto read_b = [&](int slot, int ks, int j) {
        if constexpr (B_KM) return read_tr(lds + slot * TILE_ELEMS + ks * 16 * 256 + b_km[j]);
        else return *reinterpret_cast<const bf16x8*>(lds + slot * TILE_ELEMS + (b_base ^ (ks * 16)) + j * 32 * BK);
    };

    // One k-step: 8 MFMAs on (ac, bc) with the 6 fragment reads of the following k-step (from slots
    // sa_n / sb_n at k-step ks_n) and this k-step's share of the global->LDS loads placed between
    // them one by one.  Nothing may move across the scheduling barriers: loads issued back to back
    // hold up the wave's MFMA issue, and a fragment read issued ahead of the first MFMA would be
    // waited for together with the current fragments (a full LDS round trip with the matrix pipe
    // idle).
    bf16x8 a0[2], b0[4], a1[2], b1[4];
#define OI_KSTEP(ac, bc, an, bn, sa_n, sb_n, ks_n, LOADS_AT)                                                     \
    {                                                                                                            \
        _Pragma("unroll") for (int q = 0; q < 8; ++q) {                                                          \
            acc[q >> 2][q & 3] =                                                                                 \
                __builtin_amdgcn_mfma_f32_32x32x16_bf16(ac[q >> 2], bc[q & 3], acc[q >> 2][q & 3], 0, 0, 0);     \
            __builtin_amdgcn_sched_barrier(0);                                                                   \
            LOADS_AT(q)                                                                                          \
            if (q < 2) an[q] = read_a(sa_n, ks_n, q);                                                            \
            else if (q < 6) bn[q - 2] = read_b(sb_n, ks_n, q - 2);                                               \
            __builtin_amdgcn_sched_barrier(0);                                                                   \
        }                                                                                                        \
    }
    // the 8 loads of a k-tile iteration, as evenly spread as the slot hand-over allows; OFF selects
    // the lanes' offsets (off, or last when the k-tile being fetched is the last one)
#define OI_LOADS_KS0(q)                                         \
    if (q == 1) load_block(lb, b_n1, lb.off[3], s_b1, 3);       \
    if (q == 5) load_block(la, a_n2, la.OFF2[0], s_a2, 0);
#define OI_LOADS_KS1(q) \
    if (q == 3) load_block(la, a_n2, la.OFF2[1], s_a2, 1);
#define OI_LOADS_KS2(q)                                         \
    if (q == 1) load_block(la, a_n2, la.OFF2[2], s_a2, 2);      \
    if (q == 5) load_block(la, a_n2, la.OFF2[3], s_a2, 3);
#define OI_LOADS_KS3(q)                                         \
    if (q == 0) load_block(lb, b_n2, lb.OFF2[0], s_a, 0);       \
    if (q == 3) load_block(lb, b_n2, lb.OFF2[1], s_a, 1);       \
    if (q == 6) load_block(lb, b_n2, lb.OFF2[2], s_a, 2);
#define OI_LOADS_NONE(q)
#define OI_LOADS_KS0_ONLY_B(q) \
    if (q == 1) load_block(lb, b_n1, lb.last[3], s_b1, 3);

    // A_0 and B_0 must have landed.  The wait is for everything in flight, not for "all but the 7
    // younger loads": a workgroup that runs several tiles may still have the previous tile's
    // stores outstanding, and stores complete out of order with loads.
    wait_loads_and_barrier<0>();
#pragma unroll
    for (int i = 0; i < 2; ++i) a0[i] = read_a(0, 0, i);
#pragma unroll
    for (int j = 0; j < 4; ++j) b0[j] = read_b(1, 0, j);

    // One k-tile iteration.  The last two iterations have no later k-tiles to fetch: they run
    // without those loads (no wasted traffic, nothing to drain before the epilogue).
#define OI_KTILE(L0, L1, L2, L3, PENDING)                                                                       \
    {                                                                                                            \
        const int s_a = sa, s_b = ring_slot(sa + 1);                  /* being read */                          \
        const int s_a1 = ring_slot(sa + 2), s_b1 = ring_slot(sa + 3); /* k-tile kt+1 */                         \
        const int s_a2 = ring_slot(sa + 4);                           /* free all along: takes A_(kt+2) */      \
        const char* b_n1 = k_src(lb, kt + 1);                                                                    \
        const char* a_n2 = k_src(la, kt + 2);                                                                    \
        const char* b_n2 = k_src(lb, kt + 2);                                                                    \
        (void)s_a2; (void)s_b1; (void)b_n1; (void)a_n2; (void)b_n2;                                              \
        OI_KSTEP(a0, b0, a1, b1, s_a, s_b, 1, L0)                                                                \
        OI_KSTEP(a1, b1, a0, b0, s_a, s_b, 2, L1)                                                                \
        OI_KSTEP(a0, b0, a1, b1, s_a, s_b, 3, L2)                                                                \
        /* k-tile kt+1 must have landed (its last load was issued in the first k-step above; the  */            \
        /* PENDING younger ones may stay in flight) and this wave's reads of k-tile kt must be     */            \
        /* complete: after the barrier A_kt's slot is overwritten with B_(kt+2)                    */            \
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(PENDING) : "memory");                                \
        __builtin_amdgcn_s_barrier();                                                                            \
        asm volatile("" ::: "memory");                                                                           \
        OI_KSTEP(a1, b1, a0, b0, s_a1, s_b1, 0, L3)                                                              \
        sa = s_a1;                                                                                               \
    }
    int sa = 0;  // slot of A_kt
    int64_t kt = 0;
#define OFF2 off
    for (; kt + 3 < ktiles; ++kt) OI_KTILE(OI_LOADS_KS0, OI_LOADS_KS1, OI_LOADS_KS2, OI_LOADS_KS3, 4)
#undef OFF2
#define OFF2 last
    if (kt + 2 < ktiles) {  // this iteration fetches the last k-tile
        OI_KTILE(OI_LOADS_KS0, OI_LOADS_KS1, OI_LOADS_KS2, OI_LOADS_KS3, 4)
        ++kt;
    }
#undef OFF2
    if (kt + 1 < ktiles) {
        OI_KTILE(OI_LOADS_KS0_ONLY_B, OI_LOADS_NONE, OI_LOADS_NONE, OI_LOADS_NONE, 0)
        ++kt;
    }
    OI_KTILE(OI_LOADS_NONE, OI_LOADS_NONE, OI_LOADS_NONE, OI_LOADS_NONE, 0)
#undef OI_KTILE
#undef OI_KSTEP
#undef OI_LOADS_KS0
#undef OI_LOADS_KS1
#undef OI_LOADS_KS2
#undef OI_LOADS_KS3
#undef OI_LOADS_NONE
#undef OI_LOADS_KS0_ONLY_B
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // every wave is done reading before the caller reuses the LDS (epilogue staging, next tile)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
// both operands k-contiguous: C[m, n] = sum_k A[m0 + m, k] * B[n0 + n, k]
__device__ __forceinline__ void gemm_tile(AccTile& acc, const uint16_t* __restrict__ A, int64_t lda, int64_t m0,
                                          int64_t M, const uint16_t* __restrict__ B, int64_t ldb, int64_t n0,
                                          int64_t N, int64_t K, uint16_t* lds) {
    const Operand a = {A, lda, m0, M, K}, b = {B, ldb, n0, N, K};
    gemm_tile<false, false>(acc, a, b, K, lds);
}

// Accumulator geometry of one wave: element (i, j, r) of lane `lane` is
//   m (row, vocabulary in the logits kernels) = wm*64 + i*32 + (r/4)*8 + (lane/32)*4 + r%4
//   n (column, token in the logits kernels)   = wn*128 + j*32 + lane%32
__device__ __forceinline__ int acc_row(int wm, int i, int r, int lane) {
    return wm * 64 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
}
__device__ __forceinline__ int acc_col(int wn, int j, int lane) { return wn * 128 + j * 32 + (lane & 31); }

// Online softmax statistics in the log2 domain of the scaled logits x = z * c:
//   m = max x,  s = sum 2^(x - m),  t = sum 2^(x - m) * (x - m)
// (entropy = ln2 * (log2 s - t / s), logsumexp = ln2 * (m + log2 s)).
__device__ __forceinline__ void merge_stats(float ma, float sa, float ta, float mb, float sb, float tb, float* m,
                                            float* s, float* t) {
    const float mn = fmaxf(ma, mb);
    const float da = ma - mn, db = mb - mn;
    const float fa = __builtin_amdgcn_exp2f(da), fb = __builtin_amdgcn_exp2f(db);
    *s = sa * fa + sb * fb;
    *t = fa * fmaf(da, sa, ta) + fb * fmaf(db, sb, tb);
    *m = mn;
}

// Fold the 32 logits that one lane holds for token column j of a finished tile into the running
// statistics.  PARTIAL handles the last vocabulary tile: rows past the vocabulary are skipped by
// predicate (weight exactly 0) instead of through a sentinel value.
// KEEP leaves 2^(x - ref) in place of every logit (0 for rows past the vocabulary): the exponentials
// of the statistics times 2^(max - ref), which the backward products can use in place of a
// recomputation.  `ref` is the token's reference exponent (the scaled logit of its own label, known
// before the tile is computed): relative to it the kept numbers stay inside the bf16 range whatever
// the magnitude of the logits, as long as the token's largest logit is less than KEEP_MAX_LOG2
// binary orders above its label's (tokens beyond that are flagged by the merge kernel and take the
// recomputing backward).
template <bool PARTIAL, bool KEEP>
__device__ __forceinline__ void stats_update(AccTile& acc, int j, int wm, int lane, int64_t m0, int64_t vocab, float c,
                                             float ref, float& st_m, float& st_s, float& st_t) {
    // the maximum is taken over the unscaled logits (c > 0) and every exponent is one fma: the new
    // maximum is the rounded product max(z) * c while the exponents are rounded once, so the largest
    // term is 2^(a few ulp) rather than exactly 1, far below the accuracy of the sums
    float zmax = OI_NEG_BIG;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            if (!PARTIAL || m0 + acc_row(wm, i, r, lane) < vocab) zmax = fmaxf(zmax, acc[i][j][r]);
    const float mn = fmaxf(st_m, fmaxf(zmax * c, OI_NEG_BIG));
    const float shift = st_m - mn;
    const float alpha = __builtin_amdgcn_exp2f(shift);
    float s = st_s * alpha;
    float t = alpha * fmaf(shift, st_s, st_t);
    const float pow2_max = KEEP ? __builtin_amdgcn_exp2f(fminf(mn - ref, 126.f)) : 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float d = fmaf(acc[i][j][r], c, -mn);
            float e = __builtin_amdgcn_exp2f(d);
            if (PARTIAL && m0 + acc_row(wm, i, r, lane) >= vocab) {
                d = 0.f;
                e = 0.f;
            }
            s += e;
            t = fmaf(e, d, t);
            if (KEEP) acc[i][j][r] = e * pow2_max;
        }
    st_m = mn;
    st_s = s;
    st_t = t;
}

// A finished tile leaves as a bf16 image [256 tokens][256 vocabulary columns] through the LDS (rows of
// STAGE_STRIDE entries; the two 8-byte halves of every 16-byte piece swapped in rows 8..15 of each
// 16, which keeps the 8-byte stores of a wave off each other's banks), and from there to global
// memory in 16-byte pieces of whole 512-byte rows.  Rows at or past rows_valid are written as zeros.
// It leaves one column group at a time: group j holds the 64 tokens wn*128 + j*32 + (0..31) of both
// wn halves with all 256 vocabulary columns (every m-wave contributes its 64), i.e. 64 whole rows of
// the image, and goes to global memory while the next group's statistics are still being computed
// (forward per slab at the Llama-3.1-8B shape: 6.32 -> 6.28 ms against the whole image at the end, and
// fewer live registers).
__device__ __forceinline__ void stage_group_bf16(const AccTile& acc, uint16_t* stage, int wm, int wn, int lane, int j) {
    asm volatile("" : "+v"(lane));
    const int nl = acc_col(wn, j, lane);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int vl = acc_row(wm, i, q * 4, lane) ^ (((nl >> 3) & 1) << 2);
            const uint2 pk = make_uint2(oi_pack_bf16x2(acc[i][j][q * 4], acc[i][j][q * 4 + 1]),
                                        oi_pack_bf16x2(acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]));
            *reinterpret_cast<uint2*>(stage + nl * STAGE_STRIDE + vl) = pk;
        }
}
__device__ __forceinline__ void copy_staged_group(const uint16_t* stage, uint16_t* __restrict__ dst, int64_t ld, int tid,
                                                  int rows_valid, int j) {
    // the lane's addresses are formed here, where they are used, not ahead of the tile's main loop
    asm volatile("" : "+v"(tid));
#pragma unroll 1
    for (int it = 0; it < 4; ++it) {
        const int cidx = tid + it * NTHREADS;
        const int r = cidx >> 5, ch = cidx & 31;                 // r: 0..63 within the group
        const int row = (r >> 5) * 128 + j * 32 + (r & 31);      // row of the image = token of the tile
        oi_u32x4 v = *reinterpret_cast<const oi_u32x4*>(stage + row * STAGE_STRIDE + ch * 8);
        if (row & 8) v = oi_u32x4{v.z, v.w, v.x, v.y};
        if (row >= rows_valid) v = oi_u32x4{0u, 0u, 0u, 0u};
        *reinterpret_cast<oi_u32x4*>(dst + (int64_t)row * ld + ch * 8) = v;
    }
}

// ---------------------------------------------------------------------------------------------
// forward: per-token softmax statistics over the vocabulary tiles of one split
// ---------------------------------------------------------------------------------------------
// CACHE: the vocabulary tiles [cache_tile0, cache_tile0 + cache_tiles) also leave 2^(z c - xref[n])
// behind as bf16, token-major [n_pad, cache_ld]; rows of tokens past the end are zero.
// What a forward launch covers and where its exponentials go.  Splits [0, long_splits) take
// tiles_per_split vocabulary tiles each, the others one.  A launch hands out the long splits
// [first, first + n_first) from one set of queues and then the short splits
// [long_splits, long_splits + n_second) from a second set.
// The cache takes the vocabulary tiles [cache_tile0, cache_tile0 + cache_tiles) as columns from 0 on;
// with skip_label the label's own entry is stored as 0 (the caller adds that term itself).
struct FwdLaunch {
    int64_t tiles_per_split, long_splits, first, n_first, n_second;
    uint16_t* ecache;
    int64_t cache_ld, cache_tile0, cache_tiles;
    int skip_label;
    const float* xref;  // per token: the exponent that the kept exponentials are relative to (null: 0)
};

template <bool CACHE>
__device__ __forceinline__ void lmhead_fwd_item(const uint16_t* __restrict__ W, const uint16_t* __restrict__ hidden,
                                                const int64_t* __restrict__ labels, int64_t n_tokens, int64_t hdim,
                                                int64_t vocab, float c, const FwdLaunch& fl, int64_t n_pad,
                                                float4* __restrict__ partial, float* __restrict__ zy, int64_t split,
                                                int64_t tt, uint16_t* lds) {
    const int64_t tiles_per_split = fl.tiles_per_split, long_splits = fl.long_splits;
    const int64_t vocab_tiles = (vocab + BM - 1) / BM;
    // the first long_splits splits take tiles_per_split vocabulary tiles each, the others one
    const bool long_item = split < long_splits;
    const int64_t vt_begin = long_item ? split * tiles_per_split : long_splits * tiles_per_split + (split - long_splits);
    int64_t vt_end = vt_begin + (long_item ? tiles_per_split : 1);
    vt_end = vt_end < vocab_tiles ? vt_end : vocab_tiles;

    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6, wm = wave & 3, wn = wave >> 2;
    const int64_t n0 = tt * BN;

    float st_m[4], st_s[4], st_t[4], ref[4];
    int lab[4];  // vocabulary ids fit 32 bits (vocab <= 2^22)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        st_m[j] = OI_NEG_BIG;
        st_s[j] = 0.f;
        st_t[j] = 0.f;
        const int64_t n = n0 + acc_col(wn, j, lane);
        int64_t y = n < n_tokens ? labels[n] : 0;
        lab[j] = (int)(y < 0 ? 0 : (y >= vocab ? vocab - 1 : y));
        ref[j] = (CACHE && fl.xref && n < n_tokens) ? fl.xref[n] : 0.f;
    }

    for (int64_t vt = vt_begin; vt < vt_end; ++vt) {
        AccTile acc;
        const int64_t m0 = vt * BM;
        gemm_tile(acc, W, hdim, m0, vocab, hidden, hdim, n0, n_tokens, hdim, lds);
        const bool partial_tile = m0 + BM > vocab;
        const bool keep_tile = CACHE && vt >= fl.cache_tile0 && vt < fl.cache_tile0 + fl.cache_tiles;
        const int wave_row0 = (int)m0 + wm * 64;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // the target logit, when its row falls into this wave's 64 rows
            const int rel = lab[j] - wave_row0;
            // register of this lane that holds the label's row, -1 when another lane or wave does
            int label_reg = -1;
            if (rel >= 0 && rel < 64) {
                const int rr = rel & 31;
                if (((rr >> 2) & 1) == (lane >> 5)) label_reg = (rel >> 5) * 16 + (rr >> 3) * 4 + (rr & 3);
            }
            if (label_reg >= 0) {
                float v = 0.f;
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (i * 16 + r == label_reg) v = acc[i][j][r];
                const int64_t n = n0 + acc_col(wn, j, lane);
                if (n < n_tokens) zy[n] = v;
            }
            if (partial_tile)
                stats_update<true, CACHE>(acc, j, wm, lane, m0, vocab, c, ref[j], st_m[j], st_s[j], st_t[j]);
            else
                stats_update<false, CACHE>(acc, j, wm, lane, m0, vocab, c, ref[j], st_m[j], st_s[j], st_t[j]);
            if (CACHE && fl.skip_label && label_reg >= 0) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (i * 16 + r == label_reg) acc[i][j][r] = 0.f;
            }
            if (CACHE && keep_tile) {
                // the operand ring is free (the product ended with a barrier); the groups use disjoint rows
                // of the image, so one barrier per group (written -> read out) is all they need
                __builtin_amdgcn_sched_barrier(0);
                stage_group_bf16(acc, lds, wm, wn, lane, j);
                __syncthreads();
                const int64_t left = n_tokens - n0;
                copy_staged_group(lds, fl.ecache + n0 * fl.cache_ld + (vt - fl.cache_tile0) * BM, fl.cache_ld, tid,
                                  (int)(left < BN ? left : BN), j);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the next tile's first loads must wait until the image has been read out again
        if (CACHE && keep_tile) __syncthreads();
    }

    // merge the two lane halves (same token, other rows), then the four m-waves through LDS
    float* red = reinterpret_cast<float*>(lds);  // [4 wm][256 tokens][3]
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float om = __shfl_xor(st_m[j], 32, OI_WAVE), os = __shfl_xor(st_s[j], 32, OI_WAVE),
                    ot = __shfl_xor(st_t[j], 32, OI_WAVE);
        float mn, s, t;
        merge_stats(st_m[j], st_s[j], st_t[j], om, os, ot, &mn, &s, &t);
        if (lane < 32) {
            float* p = red + (wm * 256 + acc_col(wn, j, lane)) * 3;
            p[0] = mn;
            p[1] = s;
            p[2] = t;
        }
    }
    __syncthreads();
    if (tid < 256) {
        float m = red[tid * 3], s = red[tid * 3 + 1], t = red[tid * 3 + 2];
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            const float* p = red + (w * 256 + tid) * 3;
            merge_stats(m, s, t, p[0], p[1], p[2], &m, &s, &t);
        }
        const int64_t n = n0 + tid;
        if (n < n_tokens) partial[split * n_pad + n] = make_float4(m, s, t, 0.f);
    }
}

template <bool CACHE>
__global__ void __launch_bounds__(NTHREADS)
    lmhead_fwd_kernel(const uint16_t* __restrict__ W, const uint16_t* __restrict__ hidden,
                      const int64_t* __restrict__ labels, int64_t n_tokens, const int32_t* __restrict__ n_dev,
                      int64_t hdim, int64_t vocab, float c, FwdLaunch fl, int64_t n_pad, float4* __restrict__ partial,
                      float* __restrict__ zy, uint32_t* __restrict__ queue) {
    __shared__ __align__(16) uint16_t lds[LDS_ELEMS];
    if (n_dev) n_tokens = *n_dev;  // rows selected on the device: the host only knows an upper bound
    const int64_t token_tiles = (n_tokens + BN - 1) / BN;
    // every long item of every XCD's queue is taken before the first short one: the short items are
    // there to fill the end of the launch
    for_each_tile(queue, fl.n_first, token_tiles, lds, [&](int64_t split, int64_t tt) {
        lmhead_fwd_item<CACHE>(W, hidden, labels, n_tokens, hdim, vocab, c, fl, n_pad, partial, zy, fl.first + split, tt,
                               lds);
    });
    for_each_tile(queue + QUEUE_WORDS, fl.n_second, token_tiles, lds, [&](int64_t split, int64_t tt) {
        lmhead_fwd_item<CACHE>(W, hidden, labels, n_tokens, hdim, vocab, c, fl, n_pad, partial, zy,
                               fl.long_splits + split, tt, lds);
    });
}

// A token whose largest scaled logit lies more than this many binary orders above its reference
// exponent is not served from kept exponentials (they would leave the bf16 range, or the factor
// that undoes the reference would): 2^64 leaves room for the fp32 sums over the vocabulary above it
// and for the per-token factor 2^(ref - lse2) >= 2^-(64 + 22) below it.
constexpr float KEEP_MAX_LOG2 = 64.f;

// Merges the partial statistics of token n over the vocabulary splits.  With a row selection
// (`rows` non-null) token n of the compacted batch is row rows[n] of the caller's tensors, the count
// comes from the device, and the rows that were left out are written as zeros: the grid covers
// n_total rows, thread i handles compacted token i and caller row i.
// `unsafe` (one byte per caller row, optional, cleared by the caller beforehand): set for a token
// whose kept exponentials cannot be trusted (its maximum is too far above xref[n], or is not a
// number); never cleared here, so marks that the caller has put there survive.
// Launch: 256 threads = 4 waves; a workgroup handles 64 tokens (lane = token, so the 16-byte partials
// of a split are read as one contiguous piece per wave), wave w merges the splits w, w + 4, ... and
// the four results meet in the LDS.
constexpr int COMBINE_TOKENS = 64;
__global__ void __launch_bounds__(256)
    lmhead_fwd_combine_kernel(const float4* __restrict__ partial, const float* __restrict__ zy, int64_t n_tokens,
                              const int32_t* __restrict__ n_dev, const int32_t* __restrict__ rows,
                              const uint8_t* __restrict__ row_mask, int64_t n_total, int64_t n_splits, int64_t n_pad,
                              float inv_t, float c, float* __restrict__ logprob, float* __restrict__ entropy,
                              float* __restrict__ lse_out, const float* __restrict__ xref,
                              uint8_t* __restrict__ unsafe) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t n = (int64_t)blockIdx.x * COMBINE_TOKENS + lane;
    if (n_dev) n_tokens = *n_dev;
    if (wave == 0 && row_mask && n < n_total && !row_mask[n]) {
        logprob[n] = 0.f;
        if (entropy) entropy[n] = 0.f;
        if (lse_out) lse_out[n] = 0.f;
    }
    float m = OI_NEG_BIG, s = 0.f, t = 0.f;
    if (n < n_tokens)
        for (int64_t sp = wave; sp < n_splits; sp += 4) {
            const float4 p = partial[sp * n_pad + n];
            merge_stats(m, s, t, p.x, p.y, p.z, &m, &s, &t);
        }
    __shared__ float red[3][3][COMBINE_TOKENS];
    if (wave > 0) {
        red[wave - 1][0][lane] = m;
        red[wave - 1][1][lane] = s;
        red[wave - 1][2][lane] = t;
    }
    __syncthreads();
    if (wave != 0 || n >= n_tokens) return;
#pragma unroll
    for (int w = 0; w < 3; ++w) merge_stats(m, s, t, red[w][0][lane], red[w][1][lane], red[w][2][lane], &m, &s, &t);
    const double ln2 = 0.69314718055994530942;
    const double log2s = log2((double)s);
    // the statistics are in units of x = z * c with the fp32 constant c the tile kernel multiplied by:
    // back to nats through that very constant (inv_t / c, not the literal ln 2), so that the logprob of
    // a token whose label holds all of the probability comes out as 0 at any size of the logits
    const double lse = ((double)m + log2s) * ((double)inv_t / (double)c);
    const int64_t o = rows ? rows[n] : n;
    logprob[o] = (float)((double)zy[n] * (double)inv_t - lse);
    if (entropy) entropy[o] = (float)((log2s - (double)t / (double)s) * ln2);
    if (lse_out) lse_out[o] = (float)lse;
    if (unsafe && !(m - (xref ? xref[n] : 0.f) <= KEEP_MAX_LOG2)) unsafe[o] = 1;  // a NaN maximum is flagged too
}

// ---------------------------------------------------------------------------------------------
// backward step 1: dZ tile = g * inv_T * (onehot - softmax), bf16, both orientations
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void lmhead_dz_tile(const uint16_t* __restrict__ W, const uint16_t* __restrict__ hidden,
                                               const int64_t* __restrict__ labels, const float* __restrict__ lse,
                                               const float* __restrict__ grad, const float* __restrict__ logprob,
                                               int64_t n_tokens, int64_t hdim, int64_t vocab, float c, float inv_t,
                                               int64_t v_begin, int64_t chunk_cols, int64_t n_pad,
                                               uint16_t* __restrict__ dz, int64_t vt, int64_t tt, uint16_t* lds) {
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6, wm = wave & 3, wn = wave >> 2;
    const int64_t n0 = tt * BN, m0 = v_begin + vt * BM;

    AccTile acc;
    gemm_tile(acc, W, hdim, m0, vocab, hidden, hdim, n0, n_tokens, hdim, lds);

    // stage[n][v]: rows = tokens of the tile, 256 (+8 pad) vocabulary columns.  A lane stores 8 bytes
    // (4 vocabulary entries of one token) and consecutive lanes store to consecutive rows, 132 words
    // apart: the stores of rows 8 apart meet on the same banks (measured: 1000 conflict cycles per
    // tile).  Rows 8..15 of every 16 therefore swap the two 8-byte halves of each 16-byte piece
    // (0 conflict cycles); the copy-out swaps them back.
    uint16_t* stage = lds;
    const int rows_left = (int)(vocab - m0 < BM ? vocab - m0 : BM);  // real vocabulary rows of the tile
    const int wave_row0 = wm * 64;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int nl = acc_col(wn, j, lane);
        const int64_t n = n0 + nl;
        const bool live = n < n_tokens;
        const float g = live ? grad[n] * inv_t : 0.f;
        // a token without gradient gets an exponent of -huge: every entry becomes -0 * 0
        const float l2 = g != 0.f ? lse[n] * OI_LOG2E : 3.0e38f;
        int64_t y = live ? labels[n] : -1;
        if (live) y = y < 0 ? 0 : (y >= vocab ? vocab - 1 : y);
        // The label's entry is g (1 - p_label) = - g expm1(logprob), taken from the forward's result
        // (exact also where p_label is close to 1) and written over the entry that the sweep below
        // leaves there: the sweep itself then treats all entries alike.
        const int rel = (live && y >= m0 && y < m0 + BM) ? (int)(y - m0) - wave_row0 : -1;
        const bool mine = rel >= 0 && rel < 64 && (((rel & 31) >> 2) & 1) == (lane >> 5);
        const float ng = -g;
        auto sweep = [&](auto last_tile_tag) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float d[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = q * 4 + e;
                        float val = ng * __builtin_amdgcn_exp2f(fmaf(acc[i][j][r], c, -l2));
                        if (decltype(last_tile_tag)::value && acc_row(wm, i, r, lane) >= rows_left) val = 0.f;
                        d[e] = val;
                    }
                    const int vl = acc_row(wm, i, q * 4, lane) ^ (((nl >> 3) & 1) << 2);
                    uint2 pk = make_uint2(oi_pack_bf16x2(d[0], d[1]), oi_pack_bf16x2(d[2], d[3]));
                    *reinterpret_cast<uint2*>(stage + nl * STAGE_STRIDE + vl) = pk;
                }
        };
        if (rows_left < BM) sweep(std::true_type{});  // the last vocabulary tile: rows past the vocabulary hold 0
        else sweep(std::false_type{});
        if (mine) {
            // same lane, same LDS word as the store above: program order keeps them apart
            const float val = ng * expm1f(logprob[n]);
            stage[nl * STAGE_STRIDE + ((wave_row0 + rel) ^ (((nl >> 3) & 1) << 2))] = (uint16_t)oi_f32_to_bf16_bits(val);
        }
    }
    __syncthreads();
    const int64_t vcol0 = vt * BM;  // column of this tile inside the chunk
    // [token, vocab] order: 32 16-byte pieces per token row
#pragma unroll 4
    for (int it = 0; it < 16; ++it) {
        const int cidx = tid + it * NTHREADS;
        const int row = cidx >> 5, ch = cidx & 31;
        oi_u32x4 v = *reinterpret_cast<const oi_u32x4*>(stage + row * STAGE_STRIDE + ch * 8);
        if (row & 8) v = oi_u32x4{v.z, v.w, v.x, v.y};
        *reinterpret_cast<oi_u32x4*>(dz + (n0 + row) * chunk_cols + vcol0 + ch * 8) = v;
    }
}

__global__ void __launch_bounds__(NTHREADS)
    lmhead_dz_kernel(const uint16_t* __restrict__ W, const uint16_t* __restrict__ hidden,
                     const int64_t* __restrict__ labels, const float* __restrict__ lse,
                     const float* __restrict__ grad, const float* __restrict__ logprob, int64_t n_tokens,
                     const int32_t* __restrict__ n_dev, int64_t hdim, int64_t vocab, float c, float inv_t,
                     int64_t v_begin, int64_t chunk_cols, int64_t n_pad, uint16_t* __restrict__ dz,
                     uint32_t* __restrict__ queue) {
    __shared__ __align__(16) uint16_t lds[LDS_ELEMS];
    if (n_dev) {
        n_tokens = *n_dev;
        n_pad = (n_tokens + BN - 1) / BN * BN;
    }
    for_each_tile(queue, chunk_cols / BM, n_pad / BN, lds, [&](int64_t vt, int64_t tt) {
        lmhead_dz_tile(W, hidden, labels, lse, grad, logprob, n_tokens, hdim, vocab, c, inv_t, v_begin, chunk_cols, n_pad, dz,
                       vt, tt, lds);
    });
}

// ---------------------------------------------------------------------------------------------
// backward steps 2 and 3: plain tile products with a store epilogue
// ---------------------------------------------------------------------------------------------
// Transposes the 4 x 4 block that a quad of lanes holds: on entry lane k of the quad has v[e] = M[e][k]
// (one column, four consecutive rows, which is how the MFMA leaves its results), on return
// v[f] = M[k][f] (one row, four consecutive columns, which is what a 16-byte store wants).  Two
// exchange steps inside the quad (DPP), every lane of the wave must take part.
__device__ __forceinline__ float quad_swap(float x, bool far) {
    const int i = __float_as_int(x);
    return __int_as_float(far ? __builtin_amdgcn_mov_dpp(i, 0x4E /* quad_perm 2,3,0,1 */, 0xF, 0xF, true)
                              : __builtin_amdgcn_mov_dpp(i, 0xB1 /* quad_perm 1,0,3,2 */, 0xF, 0xF, true));
}
__device__ __forceinline__ void quad_transpose(float (&v)[4], int lane) {
    const bool b0 = lane & 1, b1 = lane & 2;
    const float r01 = quad_swap(b0 ? v[0] : v[1], false), r23 = quad_swap(b0 ? v[2] : v[3], false);
    const float t0 = b0 ? r01 : v[0], t1 = b0 ? v[1] : r01, t2 = b0 ? r23 : v[2], t3 = b0 ? v[3] : r23;
    const float ra = quad_swap(b1 ? t0 : t2, true), rb = quad_swap(b1 ? t1 : t3, true);
    v[0] = b1 ? ra : t0;
    v[1] = b1 ? rb : t1;
    v[2] = b1 ? t2 : ra;
    v[3] = b1 ? t3 : rb;
}

// mode 0: out_f32  = acc          mode 1: out_f32 += acc
// mode 2: out_bf16 = acc          mode 3: out_bf16 = out_f32 + acc   (last chunk of d_hidden)
// mode 4: out_bf16 += acc         (rows added to a d_weight that was already rounded)
// A, B: operands without their tile origin (r0 is filled in here); the product has M x N
// entries, of which rows below m_valid are stored.  K == 0 stores zeros.  With `out_rows`, row r
// of a bf16 result goes to row out_rows[r] of out_bf16 (the fp32 accumulator stays compact).
template <bool A_KM, bool B_KM>
__device__ __forceinline__ void gemm_store_tile(Operand A, int64_t M, Operand B, int64_t N, int64_t K, int mode,
                                                float* out_f32, uint16_t* out_bf16, int64_t ldo, int64_t m_valid,
                                                const int32_t* __restrict__ out_rows,
                                                const float* __restrict__ scale_a, const float* __restrict__ scale_b,
                                                int64_t tm, int64_t tn, uint16_t* lds) {
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6, wm = wave & 3, wn = wave >> 2;
    const int64_t m0 = tm * BM, n0 = tn * BN;
    A.r0 = m0;
    B.r0 = n0;
    AccTile acc;
    if (K <= 0 && (mode == 1 || mode == 4)) return;  // nothing to add
    if (K > 0) {
        gemm_tile<A_KM, B_KM>(acc, A, B, K, lds);
    } else {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    }
    if (((N | ldo) & 3) == 0 && (reinterpret_cast<uintptr_t>(out_f32) & 15) == 0 &&
        (reinterpret_cast<uintptr_t>(out_bf16) & 7) == 0) {
        // Every store and load of the epilogue as a 16-byte piece (8 bytes of bf16): after a 4 x 4
        // transpose inside each quad of lanes a lane holds four consecutive columns of one row.  A
        // quarter of the memory instructions of the one-value-per-lane form, whose address
        // processing is what an epilogue of 128 values per lane waits for.  The fp32 sum of the
        // accumulating modes is requested before the transposes of the half tile it belongs to and
        // added with plain loads and stores: every element has one writer per launch and the
        // launches follow each other on the stream, so no atomic is needed.
        const int kq = lane & 3, g = (lane & 31) >> 2, hl = lane >> 5;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            int64_t row[4], dst[4];
            bool ok[4];
            float sa[4], sb[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                row[q] = m0 + wm * 64 + i * 32 + q * 8 + hl * 4 + kq;
                ok[q] = row[q] < m_valid;
                dst[q] = (ok[q] && out_rows) ? (int64_t)out_rows[row[q]] : row[q];
                sa[q] = (ok[q] && scale_a) ? scale_a[row[q]] : 1.f;
                sb[q] = (ok[q] && scale_a) ? scale_b[row[q]] : 1.f;
            }
            // two of the four 32-column blocks at a time: 32 registers of sums in flight
#pragma unroll
            for (int jh = 0; jh < 2; ++jh) {
                oi_f32x4 part[2][4];
                uint2 part16[2][4];
                if (mode == 1 || mode == 3) {
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int64_t col = n0 + wn * 128 + (2 * jh + jj) * 32 + 4 * g;
                            part[jj][q] = (ok[q] && col < N)
                                              ? *reinterpret_cast<const oi_f32x4*>(out_f32 + row[q] * ldo + col)
                                              : oi_f32x4{0.f, 0.f, 0.f, 0.f};
                        }
                } else if (mode == 4) {
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int64_t col = n0 + wn * 128 + (2 * jh + jj) * 32 + 4 * g;
                            part16[jj][q] = (ok[q] && col < N)
                                                ? *reinterpret_cast<const uint2*>(out_bf16 + dst[q] * ldo + col)
                                                : make_uint2(0u, 0u);
                        }
                }
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    const int j = 2 * jh + jj;
                    const int64_t col = n0 + wn * 128 + j * 32 + 4 * g;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float v[4] = {acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
                        quad_transpose(v, lane);
                        if (!ok[q] || col >= N) continue;
                        if (scale_a) {
                            // a row whose factor is exactly 0 is 0 whatever its sum holds (the sums of
                            // rows that were taken out may have left the fp32 range)
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] = sb[q] == 0.f ? 0.f : v[e] * sa[q] * sb[q];
                        }
                        if (mode == 1 || mode == 3) {
                            v[0] += part[jj][q].x;
                            v[1] += part[jj][q].y;
                            v[2] += part[jj][q].z;
                            v[3] += part[jj][q].w;
                        } else if (mode == 4) {
                            v[0] += oi_bf16lo_to_f32(part16[jj][q].x);
                            v[1] += oi_bf16hi_to_f32(part16[jj][q].x);
                            v[2] += oi_bf16lo_to_f32(part16[jj][q].y);
                            v[3] += oi_bf16hi_to_f32(part16[jj][q].y);
                        }
                        if (mode <= 1)
                            *reinterpret_cast<oi_f32x4*>(out_f32 + row[q] * ldo + col) = oi_f32x4{v[0], v[1], v[2], v[3]};
                        else
                            *reinterpret_cast<uint2*>(out_bf16 + dst[q] * ldo + col) =
                                make_uint2(oi_pack_bf16x2(v[0], v[1]), oi_pack_bf16x2(v[2], v[3]));
                    }
                }
            }
        }
        return;
    }
    if (mode >= 2 && (ldo & 1) == 0) {
        // bf16 output: neighbouring lanes hold neighbouring columns of the same rows; after one DPP
        // swap per pair of rows every lane stores two columns of one row as a 4-byte word (half as
        // many, twice as wide stores as one bf16 per lane)
        const bool odd = lane & 1;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int64_t row = m0 + acc_row(wm, i, 2 * t, lane) + (odd ? 1 : 0);
                // a lane past the last row still takes part in the exchange below: its neighbour
                // holds the row before it and needs this lane's half of that row
                const bool row_ok = row < m_valid;
                const int64_t dst_row = (row_ok && out_rows) ? (int64_t)out_rows[row] : row;
                const float sa = (row_ok && scale_a) ? scale_a[row] : 1.f, sb = (row_ok && scale_a) ? scale_b[row] : 1.f;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int64_t col = n0 + (acc_col(wn, j, lane) & ~1);
                    const float own0 = acc[i][j][2 * t], own1 = acc[i][j][2 * t + 1];
                    const float send = odd ? own0 : own1;
                    const float recv = __int_as_float(
                        __builtin_amdgcn_mov_dpp(__float_as_int(send), 0xB1 /* quad_perm 1,0,3,2 */, 0xF, 0xF, true));
                    float lo = odd ? recv : own0, hi = odd ? own1 : recv;
                    if (!row_ok || col >= N) continue;
                    if (scale_a) {
                        // a row whose factor is exactly 0 is 0 whatever its sum holds (the sums of
                        // rows that were taken out may have left the fp32 range)
                        lo = sb == 0.f ? 0.f : lo * sa * sb;
                        hi = sb == 0.f ? 0.f : hi * sa * sb;
                    }
                    const int64_t o = row * ldo + col, d = dst_row * ldo + col;
                    if (col + 1 < N) {
                        if (mode == 3) {
                            const float2 part = *reinterpret_cast<const float2*>(out_f32 + o);
                            lo += part.x;
                            hi += part.y;
                        } else if (mode == 4) {
                            const uint32_t prev = *reinterpret_cast<const uint32_t*>(out_bf16 + d);
                            lo += oi_bf16lo_to_f32(prev);
                            hi += oi_bf16hi_to_f32(prev);
                        }
                        *reinterpret_cast<uint32_t*>(out_bf16 + d) = oi_pack_bf16x2(lo, hi);
                    } else {
                        if (mode == 3) lo += out_f32[o];
                        else if (mode == 4) lo += oi_bf16lo_to_f32((uint32_t)out_bf16[d]);
                        out_bf16[d] = (uint16_t)oi_f32_to_bf16_bits(lo);
                    }
                }
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t col = n0 + acc_col(wn, j, lane);
            if (col >= N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t row = m0 + acc_row(wm, i, r, lane);
                if (row >= m_valid) continue;
                const int64_t o = row * ldo + col;
                float v = acc[i][j][r];
                if (scale_a) v = scale_b[row] == 0.f ? 0.f : v * scale_a[row] * scale_b[row];
                if (mode == 1) {
                    // the addition is done by the L2 (no load to wait for: 8.2 -> 6.9 ms per d_weight slab product);
                    // every element has one writer per launch and the launches follow each other on
                    // the stream, so the sum is the one a load + add + store would give, to the bit
                    unsafeAtomicAdd(out_f32 + o, v);
                    continue;
                }
                if (mode == 3) v += out_f32[o];
                if (mode == 0) {
                    out_f32[o] = v;
                    continue;
                }
                const int64_t d = (out_rows ? (int64_t)out_rows[row] : row) * ldo + col;
                if (mode == 4) v += oi_bf16lo_to_f32((uint32_t)out_bf16[d]);
                out_bf16[d] = (uint16_t)oi_f32_to_bf16_bits(v);
            }
        }
}

// Sizes that depend on a row count which only the device knows (rows selected by a mask).
//   role 1 (d_hidden = dZ * W, rows of the product are tokens):  M, m_valid and A's extent follow n
//   role 2 (d_weight = dZ^T * hidden, the k dimension is tokens): K and the operands' k extents follow n
struct DynRows {
    const int32_t* n_dev;
    int role;
    const int32_t* out_rows;
    // optional factors of row r of the product, applied as (acc * scale_a[r]) * scale_b[r] before it
    // is stored or accumulated (two factors so that neither has to leave the fp32 range)
    const float *scale_a, *scale_b;
    // optional: the store mode comes from device memory (a negative value: the launch does nothing)
    const int32_t* mode_dev;
};

// `queue` null: one workgroup per tile id (blockIdx); otherwise a launch of resident workgroups
// that draw their tiles from the queue
template <bool A_KM, bool B_KM>
__global__ void __launch_bounds__(NTHREADS)
    gemm_store_kernel(Operand A, int64_t M, Operand B, int64_t N, int64_t K, int mode, float* out_f32,
                      uint16_t* out_bf16, int64_t ldo, int64_t m_valid, DynRows dyn, uint32_t* __restrict__ queue) {
    __shared__ __align__(16) uint16_t lds[LDS_ELEMS];
    if (dyn.mode_dev) {
        mode = *dyn.mode_dev;
        if (mode < 0) return;
    }
    if (dyn.n_dev) {
        const int64_t n = *dyn.n_dev;
        if (dyn.role == 1) {
            M = (n + BM - 1) / BM * BM;
            m_valid = n;
            A.extent = M;
        } else if (dyn.role == 2) {
            K = (n + BK - 1) / BK * BK;
            A.k_valid = (n + BM - 1) / BM * BM;
            B.k_valid = n;
        }
    }
    // a product without terms that would only be added changes nothing: no tile is drawn at all
    if (K <= 0 && (mode == 1 || mode == 4)) return;
    const int64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    if (queue) {
        for_each_tile(queue, tiles_m, tiles_n, lds, [&](int64_t tm, int64_t tn) {
            gemm_store_tile<A_KM, B_KM>(A, M, B, N, K, mode, out_f32, out_bf16, ldo, m_valid, dyn.out_rows, dyn.scale_a,
                                        dyn.scale_b, tm, tn, lds);
        });
    } else {
        int64_t tm, tn;
        if (tile_of_block(tiles_m, tiles_n, &tm, &tn))
            gemm_store_tile<A_KM, B_KM>(A, M, B, N, K, mode, out_f32, out_bf16, ldo, m_valid, dyn.out_rows, dyn.scale_a,
                                        dyn.scale_b, tm, tn, lds);
    }
}

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

__global__ void zero_words_kernel(uint32_t* __restrict__ p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}
__global__ void zero_bytes_kernel(uint8_t* __restrict__ p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// ---------------------------------------------------------------------------------------------
// row selection: which token rows are multiplied at all
// ---------------------------------------------------------------------------------------------
// Row i takes part when its mask byte is set (no mask: every row) and, in the backward pass when
// asked for, when its upstream gradient is not exactly zero.  The selection is made on the device
// and stays there: the host sizes grids and buffers for all n rows and every kernel reads the
// selected count from memory, so no call ever waits for the GPU.
__device__ __forceinline__ bool row_selected(const uint8_t* __restrict__ mask, const float* __restrict__ grad,
                                             int64_t i) {
    return (!mask || mask[i] != 0) && (!grad || grad[i] != 0.f);
}

constexpr int SELECT_THREADS = 1024;
// One workgroup: rows[0 .. count) = positions of the selected rows in ascending order (a stable
// compaction: count per thread segment, block scan, write).  Also clears `n_zero` (<= 1024) queue
// words for the launches that follow.
__global__ void __launch_bounds__(SELECT_THREADS)
    select_rows_kernel(const uint8_t* __restrict__ mask, const float* __restrict__ grad, int64_t n,
                       int32_t* __restrict__ rows, int32_t* __restrict__ count, uint32_t* __restrict__ zero_words,
                       int n_zero) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int64_t per = (n + SELECT_THREADS - 1) / SELECT_THREADS;
    const int64_t b = t * per, e = b + per < n ? b + per : n;
    int c = 0;
    for (int64_t i = b; i < e; ++i) c += row_selected(mask, grad, i) ? 1 : 0;
    int incl = c;
#pragma unroll
    for (int off = 1; off < OI_WAVE; off <<= 1) {
        const int o = __shfl_up(incl, off, OI_WAVE);
        if (lane >= off) incl += o;
    }
    __shared__ int wave_total[SELECT_THREADS / OI_WAVE];
    if (lane == OI_WAVE - 1) wave_total[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += wave_total[w];
    int pos = base + incl - c;
    for (int64_t i = b; i < e; ++i)
        if (row_selected(mask, grad, i)) rows[pos++] = (int32_t)i;
    if (t == SELECT_THREADS - 1) *count = base + incl;
    if (t < n_zero) zero_words[t] = 0u;
}

// Workgroup j copies selected row j: the hidden-state row (hdim bf16, 16-byte pieces), its label
// and, for the backward pass, its logsumexp and upstream gradient.
__global__ void __launch_bounds__(256)
    gather_rows_kernel(const uint16_t* __restrict__ hidden, const int64_t* __restrict__ labels,
                       const float* __restrict__ lse, const float* __restrict__ grad,
                       const float* __restrict__ logprob, const int32_t* __restrict__ rows,
                       const int32_t* __restrict__ count, int64_t hdim, uint16_t* __restrict__ hidden_c,
                       int64_t* __restrict__ labels_c, float* __restrict__ lse_c, float* __restrict__ grad_c,
                       float* __restrict__ logprob_c) {
    const int64_t j = blockIdx.x;
    if (j >= *count) return;
    const int64_t src = rows[j];
    const oi_u32x4* from = reinterpret_cast<const oi_u32x4*>(hidden + src * hdim);
    oi_u32x4* to = reinterpret_cast<oi_u32x4*>(hidden_c + j * hdim);
    for (int64_t c = threadIdx.x; c < hdim / 8; c += blockDim.x) to[c] = from[c];
    if (threadIdx.x == 0) {
        labels_c[j] = labels[src];
        if (lse_c) lse_c[j] = lse[src];
        if (grad_c) grad_c[j] = grad[src];
        if (logprob_c) logprob_c[j] = logprob[src];
    }
}

// xref[j] = c * <hidden[j, :], W[label_j, :]>: the scaled logit of token j's own label, the exponent
// that the token's kept exponentials are relative to.  It needs to be close to the token's largest
// scaled logit, not equal to it (the same number is taken out again wherever the exponentials are
// used), so the summation order of this dot product does not matter.  One wave per token.
__global__ void __launch_bounds__(256)
    label_ref_kernel(const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ W,
                     const int64_t* __restrict__ labels, const int32_t* __restrict__ n_dev, int64_t n_tokens,
                     int64_t hdim, int64_t vocab, float c, float* __restrict__ xref) {
    const int lane = threadIdx.x & 63;
    const int64_t j = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n_dev) n_tokens = *n_dev;
    if (j >= n_tokens) return;
    int64_t y = labels[j];
    y = y < 0 ? 0 : (y >= vocab ? vocab - 1 : y);
    const oi_u32x4* a = reinterpret_cast<const oi_u32x4*>(hidden + j * hdim);
    const oi_u32x4* b = reinterpret_cast<const oi_u32x4*>(W + y * hdim);
    float acc = 0.f;
    for (int64_t p = lane; p < hdim / 8; p += OI_WAVE) {  // hdim is a multiple of 64
        const oi_u32x4 av = a[p], bv = b[p];
        const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            acc = fmaf(oi_bf16lo_to_f32(aw[k]), oi_bf16lo_to_f32(bw[k]), acc);
            acc = fmaf(oi_bf16hi_to_f32(aw[k]), oi_bf16hi_to_f32(bw[k]), acc);
        }
    }
    acc = oi_wave_sum(acc);
    if (lane == 0) xref[j] = acc * c;
}

// Which rows a slab pass works on: rows order[offset .. offset + count) of a row index that lives
// on the device.  Written by a planning kernel, read by every kernel of the pass.
struct SlabMeta {
    int32_t offset, count;
    // how the slab's d_weight product is stored (the modes of gemm_store_tile): the only slab writes
    // bf16 rows (2); of several, the first stores fp32 (0), the middle ones add to it (1) and the last
    // one adds the fp32 sum to its own product and writes bf16 rows (3); a pass without rows: -1
    int32_t dw_mode, reserved;
};

// Workgroup j copies row order[meta->offset + j] into the slab's own buffers: the hidden-state row
// (hdim bf16, 16-byte pieces), its label, its row number and, when given, its logsumexp, upstream
// gradient and logprob.
__global__ void __launch_bounds__(256)
    gather_slab_kernel(const uint16_t* __restrict__ hidden, const int64_t* __restrict__ labels,
                       const float* __restrict__ lse, const float* __restrict__ grad,
                       const float* __restrict__ logprob, const int32_t* __restrict__ order,
                       const SlabMeta* __restrict__ meta, int64_t hdim, uint16_t* __restrict__ hidden_s,
                       int64_t* __restrict__ labels_s, int32_t* __restrict__ rows_s, float* __restrict__ lse_s,
                       float* __restrict__ grad_s, float* __restrict__ logprob_s) {
    const int64_t j = blockIdx.x;
    if (j >= meta->count) return;
    const int64_t src = order[meta->offset + j];
    const oi_u32x4* from = reinterpret_cast<const oi_u32x4*>(hidden + src * hdim);
    oi_u32x4* to = reinterpret_cast<oi_u32x4*>(hidden_s + j * hdim);
    for (int64_t c = threadIdx.x; c < hdim / 8; c += blockDim.x) to[c] = from[c];
    if (threadIdx.x == 0) {
        labels_s[j] = labels[src];
        rows_s[j] = (int32_t)src;
        if (lse_s) lse_s[j] = lse[src];
        if (grad_s) grad_s[j] = grad[src];
        if (logprob_s) logprob_s[j] = logprob[src];
    }
}

// Backward products straight from the kept exponentials e'[n, v] = 2^(x_nv - ref_n), x = z c:
//   dZ[n, v] = g_n inv_T (1[v = y_n] - 2^(x_nv - lse2_n)) = s_n (e'[n, v] - 1[v = y_n] 2^(lse2_n - ref_n)),
//   s_n = -g_n inv_T 2^(ref_n - lse2_n).
// The per-token factor leaves the products: d_hidden[n] = s_n (e'[n, :] W) (a row factor in the
// store epilogue) and d_weight = e'^T (s h) (the hidden rows are scaled once).  Workgroup j prepares
// token j of a slab (caller row rows_s[j]): the two halves of s_n (so that neither leaves the fp32
// range), the label's entry of the slab's exponentials, replaced by
// 2^(x_y - ref) - 2^(lse2 - ref) = 2^(lse2 - ref) expm1(logprob) from the forward's fp32 logprob
// (exact where the label's probability is close to 1), and, when d_weight is wanted, the scaled
// hidden row.  A token flagged in `unsafe` gets factors of exactly 0: it adds nothing to either
// product here and takes the recomputing backward afterwards.
__global__ void __launch_bounds__(256)
    slab_prepare_kernel(const float* __restrict__ lse, const float* __restrict__ grad,
                        const float* __restrict__ logprob, const uint8_t* __restrict__ unsafe,
                        const int32_t* __restrict__ rows_s, const int64_t* __restrict__ labels_s,
                        const float* __restrict__ xref_s, const SlabMeta* __restrict__ meta, float inv_t,
                        int64_t vocab, int64_t hdim, uint16_t* __restrict__ ecache, int64_t cache_ld,
                        const uint16_t* __restrict__ hidden_s, float* __restrict__ scale_a,
                        float* __restrict__ scale_b, uint16_t* __restrict__ scaled_hidden) {
    const int64_t j = blockIdx.x;
    if (j >= meta->count) return;
    const int64_t src = rows_s[j];
    const bool dead = unsafe[src] != 0;
    const float l2 = lse[src] * OI_LOG2E - xref_s[j];  // log2 of the sum of the kept numbers of this token
    const float half = dead ? 0.f : __builtin_amdgcn_exp2f(-0.5f * l2);
    const float a = half, b = -grad[src] * inv_t * half;
    if (threadIdx.x == 0) {
        scale_a[j] = a;
        scale_b[j] = b;
        int64_t y = labels_s[j];
        y = y < 0 ? 0 : (y >= vocab ? vocab - 1 : y);
        ecache[j * cache_ld + y] =
            (uint16_t)oi_f32_to_bf16_bits(__builtin_amdgcn_exp2f(fminf(l2, 126.f)) * expm1f(logprob[src]));
    }
    if (!scaled_hidden) return;
    const oi_u32x4* from = reinterpret_cast<const oi_u32x4*>(hidden_s + j * hdim);
    oi_u32x4* to = reinterpret_cast<oi_u32x4*>(scaled_hidden + j * hdim);
    for (int64_t c = threadIdx.x; c < hdim / 8; c += blockDim.x) {
        const oi_u32x4 v = from[c];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        uint32_t o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
            o[k] = dead ? 0u : oi_pack_bf16x2(oi_bf16lo_to_f32(w[k]) * a * b, oi_bf16hi_to_f32(w[k]) * a * b);
        to[c] = oi_u32x4{o[0], o[1], o[2], o[3]};
    }
}

// d_hidden rows of tokens that took no part are zero
__global__ void __launch_bounds__(256)
    zero_unselected_rows_kernel(const uint8_t* __restrict__ mask, const float* __restrict__ grad, int64_t hdim,
                                uint16_t* __restrict__ out) {
    const int64_t i = blockIdx.x;
    if (row_selected(mask, grad, i)) return;
    uint32_t* row = reinterpret_cast<uint32_t*>(out + i * hdim);  // hdim is a multiple of 64
    for (int64_t c = threadIdx.x; c < hdim / 2; c += blockDim.x) row[c] = 0u;
}

// Timing probe for the measurement harness: while armed, the slab-wise entry points record a pair
// of HIP events around every launch of one of their three tile kernels (which one is chosen when the
// probe is armed), on the stream of the call.  Off by default and between arm / read; not meant for
// calls that are being captured into a graph.
struct Probe {
    int kernel = -1;  // 0 forward with kept exponentials, 1 d_hidden product, 2 d_weight product; -1 = off
    int used = 0;
    static constexpr int MAX_LAUNCHES = 1024;
    hipEvent_t ev[2 * MAX_LAUNCHES];
};
Probe g_probe;
struct ProbeScope {
    bool on;
    hipStream_t s;
    ProbeScope(int kernel, hipStream_t stream) : on(g_probe.kernel == kernel && g_probe.used < Probe::MAX_LAUNCHES), s(stream) {
        if (on) (void)hipEventRecord(g_probe.ev[2 * g_probe.used], s);
    }
    ~ProbeScope() {
        if (on) (void)hipEventRecord(g_probe.ev[2 * g_probe.used++ + 1], s);
    }
};

// Workgroups of a queue-driven launch: one per CU of the current device (each takes a whole CU's
// LDS), a multiple of 8 so that every XCD gets the same number, and no more than there are tiles.
unsigned resident_grid(int64_t tiles_m, int64_t tiles_n) {
    const int cus = oi_cu_count();
    const int64_t grid = (cus + 7) / 8 * 8;
    const int64_t pids = pids_for_tiles(tiles_m, tiles_n);
    return (unsigned)(pids < grid ? pids : grid);
}

constexpr int64_t BWD_VOCAB_CHUNK = 32768;
// chunk of the forward that also accumulates the weighted sum of weight rows: fewer, longer launches
// (measured on the 70B head shape: 16384 columns 79.2 ms, 32768 77.3, 65536 75.4 per step)
constexpr int64_t WSUM_VOCAB_CHUNK = 65536;

struct Carver {
    size_t off = 0;
    size_t take(size_t bytes) {
        const size_t o = off;
        off += (bytes + 255) / 256 * 256;
        return o;
    }
};

// buffers of a row selection: the row index, the selected count and the compacted per-row inputs
struct SelectionPlan {
    size_t off_rows, off_count, off_hidden, off_labels, off_lse, off_grad, off_logprob;
};
SelectionPlan plan_selection(Carver& cv, int64_t n_pad, int64_t hdim, bool backward) {
    SelectionPlan p;
    p.off_rows = cv.take((size_t)n_pad * sizeof(int32_t));
    p.off_count = cv.take(sizeof(int32_t));
    p.off_hidden = cv.take((size_t)n_pad * hdim * 2);
    p.off_labels = cv.take((size_t)n_pad * sizeof(int64_t));
    p.off_lse = backward ? cv.take((size_t)n_pad * sizeof(float)) : 0;
    p.off_grad = backward ? cv.take((size_t)n_pad * sizeof(float)) : 0;
    p.off_logprob = backward ? cv.take((size_t)n_pad * sizeof(float)) : 0;
    return p;
}

// Where the forward leaves the exponentials it computes anyway (all null / 0: nowhere)
struct KeepPlan {
    uint16_t* buf;        // bf16 [n_pad, ld], token-major
    int64_t ld, tiles;    // columns of the buffer, and as vocabulary tiles
    const float* xref;    // per token: the exponent the kept numbers are relative to
    uint8_t* unsafe;      // per caller row: set when the kept numbers of that token cannot be used
};

struct FwdPlan {
    int64_t token_tiles, vocab_tiles, n_splits, tiles_per_split, long_splits, n_pad;
    int64_t chunk, n_chunks;  // chunked flavour only
    size_t off_partial, off_zy, off_queue, off_chunk, off_xref, total;
    SelectionPlan sel;
};
// `chunked`: the launch covers one backward-sized vocabulary chunk at a time (the forward that also
// accumulates the weighted sum of weight rows): every split is a long one, so that a chunk is a whole
// number of splits, and there is one set of queues per chunk for the forward and one for the product.
FwdPlan plan_fwd(int64_t n_tokens, int64_t hdim, int64_t vocab, bool with_selection, bool chunked = false) {
    FwdPlan p;
    p.token_tiles = (n_tokens + BN - 1) / BN;
    p.vocab_tiles = (vocab + BM - 1) / BM;
    p.n_pad = p.token_tiles * BN;
    // Work items of 4 vocabulary tiles (8 tiles measured 1.6 % slower, 2 tiles no faster: every
    // item also writes and later merges a set of partial statistics).  Fewer tiles per split only
    // when the problem is too small to give every CU work otherwise.
    int64_t tps = 4;
    while (tps > 1 && ((p.vocab_tiles + tps - 1) / tps) * p.token_tiles < 512) tps /= 2;
    p.tiles_per_split = tps;
    // The ids are handed out with the vocabulary split as the slow index, so the last splits are
    // the last work of the launch: they are single tiles, about four per CU, which the workgroups
    // that run out of long items pick up (the launch then ends within one tile, not one item).
    const int64_t short_wanted = (4 * 256 + p.token_tiles - 1) / p.token_tiles;
    // whole groups of 8 long splits: the ids of a group of 8 splits are handed out together, and a
    // long item among the last short ones would be the new ragged end
    p.long_splits = tps > 1 && p.vocab_tiles > short_wanted ? (p.vocab_tiles - short_wanted) / tps / 8 * 8 : 0;
    p.n_splits = p.long_splits + (p.vocab_tiles - p.long_splits * tps);
    p.chunk = p.n_chunks = 0;
    if (chunked) {
        p.n_splits = p.long_splits = (p.vocab_tiles + tps - 1) / tps;
        const int64_t v_pad = p.vocab_tiles * BM;
        p.chunk = v_pad < WSUM_VOCAB_CHUNK ? v_pad : WSUM_VOCAB_CHUNK;
        p.n_chunks = (v_pad + p.chunk - 1) / p.chunk;
    }
    Carver cv;
    p.off_partial = cv.take((size_t)p.n_splits * p.n_pad * sizeof(float4));
    p.off_zy = cv.take((size_t)p.n_pad * sizeof(float));
    p.off_queue = cv.take((chunked ? (size_t)p.n_chunks * (FWD_QUEUE_WORDS + QUEUE_WORDS) : (size_t)FWD_QUEUE_WORDS) *
                          sizeof(uint32_t));
    p.off_chunk = chunked ? cv.take((size_t)p.n_pad * p.chunk * 2) : 0;
    p.off_xref = 0;
    if (with_selection) p.sel = plan_selection(cv, p.n_pad, hdim, false);
    p.total = cv.off;
    return p;
}

struct BwdPlan {
    int64_t n_pad, v_pad, chunk, n_chunks;
    size_t off_dz, off_dh32, off_queues, total;
    SelectionPlan sel;
};
BwdPlan plan_bwd(int64_t n_tokens, int64_t hdim, int64_t vocab, bool with_selection) {
    BwdPlan p;
    p.n_pad = round_up(n_tokens, 256);
    p.v_pad = round_up(vocab, 256);
    p.chunk = p.v_pad < BWD_VOCAB_CHUNK ? p.v_pad : BWD_VOCAB_CHUNK;
    p.n_chunks = (p.v_pad + p.chunk - 1) / p.chunk;
    Carver cv;
    p.off_dz = cv.take((size_t)p.n_pad * p.chunk * 2);
    p.off_dh32 = cv.take((size_t)n_tokens * hdim * 4);
    // one set of work-queue counters per tile-kernel launch (three per vocabulary chunk)
    p.off_queues = cv.take((size_t)(3 * p.n_chunks) * QUEUE_WORDS * sizeof(uint32_t));
    if (with_selection) p.sel = plan_selection(cv, p.n_pad, hdim, true);
    p.total = cv.off;
    return p;
}

int check_lmhead(const void* hidden, const void* weight, const int64_t* labels, int64_t n_tokens, int64_t hdim,
                 int64_t vocab, float inv_t) {
    OI_RETURN_IF(n_tokens < 0 || hdim <= 0 || vocab <= 0, OI_EINVAL);
    OI_RETURN_IF(hdim % 64 != 0, OI_EINVAL);
    OI_RETURN_IF(!(inv_t >= 1.0e-6f) || !(inv_t <= 1.0e6f), OI_EINVAL);
    // row strides of every operand (hidden_dim, padded vocabulary, padded token count) are folded
    // into 32-bit byte offsets inside a 256-row tile
    OI_RETURN_IF(n_tokens > MAX_LD || vocab > MAX_LD || hdim > MAX_LD, OI_EINVAL);
    if (n_tokens == 0) return OI_OK;
    OI_RETURN_IF(!hidden || !weight || !labels, OI_ENULL);
    OI_RETURN_IF(!oi_aligned(hidden, 16) || !oi_aligned(weight, 16), OI_EALIGN);
    return OI_OK;
}

// The per-row inputs the tile kernels read: the caller's own, or their compacted copies
struct RowInputs {
    const uint16_t* hidden;
    const int64_t* labels;
    const float *lse, *grad;
    const int32_t *rows, *n_dev;  // null without a selection
    const float* logprob;         // the forward's result: the label's entry of dZ is rebuilt from it
};

// select + gather on `s`; clears `n_zero` queue words on the way
RowInputs launch_selection(const SelectionPlan& sp, char* ws, const void* hidden, const int64_t* labels,
                           const float* lse, const float* grad, const uint8_t* row_mask, bool skip_zero_grad,
                           int64_t n_tokens, int64_t hdim, uint32_t* zero_words, int n_zero, hipStream_t s,
                           const float* logprob = nullptr) {
    int32_t* rows = reinterpret_cast<int32_t*>(ws + sp.off_rows);
    int32_t* count = reinterpret_cast<int32_t*>(ws + sp.off_count);
    uint16_t* hidden_c = reinterpret_cast<uint16_t*>(ws + sp.off_hidden);
    int64_t* labels_c = reinterpret_cast<int64_t*>(ws + sp.off_labels);
    float* lse_c = lse ? reinterpret_cast<float*>(ws + sp.off_lse) : nullptr;
    float* grad_c = grad ? reinterpret_cast<float*>(ws + sp.off_grad) : nullptr;
    float* logprob_c = logprob ? reinterpret_cast<float*>(ws + sp.off_logprob) : nullptr;
    hipLaunchKernelGGL(select_rows_kernel, dim3(1), dim3(SELECT_THREADS), 0, s, row_mask,
                       skip_zero_grad ? grad : static_cast<const float*>(nullptr), n_tokens, rows, count, zero_words,
                       n_zero);
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)n_tokens), dim3(256), 0, s,
                       static_cast<const uint16_t*>(hidden), labels, lse, grad, logprob, rows, count, hdim, hidden_c,
                       labels_c, lse_c, grad_c, logprob_c);
    return RowInputs{hidden_c, labels_c, lse_c, grad_c, rows, count, logprob_c};
}

// lse, upstream gradient and logprob of the selected rows (the rows were selected and gathered earlier)
__global__ void gather_f32_kernel(const float* __restrict__ lse, const float* __restrict__ grad,
                                  const float* __restrict__ logprob, const int32_t* __restrict__ rows,
                                  const int32_t* __restrict__ count, float* __restrict__ lse_c,
                                  float* __restrict__ grad_c, float* __restrict__ logprob_c) {
    const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= *count) return;
    const int64_t src = rows[j];
    lse_c[j] = lse[src];
    grad_c[j] = grad[src];
    logprob_c[j] = logprob[src];
}

void launch_label_ref(const RowInputs& in, const void* weight, int64_t n_tokens, int64_t hidden_dim, int64_t vocab,
                      float inv_temperature, float* xref, hipStream_t s) {
    hipLaunchKernelGGL(label_ref_kernel, dim3((unsigned)((n_tokens + 3) / 4)), dim3(256), 0, s, in.hidden,
                       static_cast<const uint16_t*>(weight), in.labels, in.n_dev, n_tokens, hidden_dim, vocab,
                       inv_temperature * OI_LOG2E, xref);
}

// forward launches: tile kernel + merge of the partial statistics.  `queue` must be zeroed.
// `keep`: where the exponentials of every vocabulary tile go as well (buf null: nowhere).
void enqueue_fwd(const FwdPlan& p, char* ws, const RowInputs& in, const uint8_t* row_mask, const void* weight,
                 int64_t n_tokens, int64_t hidden_dim, int64_t vocab, float inv_temperature, float* logprob,
                 float* entropy, float* lse, const KeepPlan& keep, hipStream_t s) {
    float4* partial = reinterpret_cast<float4*>(ws + p.off_partial);
    float* zy = reinterpret_cast<float*>(ws + p.off_zy);
    uint32_t* queue = reinterpret_cast<uint32_t*>(ws + p.off_queue);
    const float c = inv_temperature * OI_LOG2E;
    const dim3 grid(resident_grid(p.n_splits, p.token_tiles));
    const uint16_t* Wp = static_cast<const uint16_t*>(weight);
    const FwdLaunch fl = {p.tiles_per_split, p.long_splits, 0, p.long_splits, p.n_splits - p.long_splits,
                          keep.buf, keep.ld, 0, keep.buf ? keep.tiles : 0, 0, keep.xref};
    if (keep.buf) {
        const ProbeScope probe(0, s);
        hipLaunchKernelGGL(lmhead_fwd_kernel<true>, grid, dim3(NTHREADS), 0, s, Wp, in.hidden, in.labels, n_tokens,
                           in.n_dev, hidden_dim, vocab, c, fl, p.n_pad, partial, zy, queue);
    } else
        hipLaunchKernelGGL(lmhead_fwd_kernel<false>, grid, dim3(NTHREADS), 0, s, Wp, in.hidden, in.labels, n_tokens,
                           in.n_dev, hidden_dim, vocab, c, fl, p.n_pad, partial, zy, queue);
    hipLaunchKernelGGL(lmhead_fwd_combine_kernel, dim3((unsigned)((n_tokens + COMBINE_TOKENS - 1) / COMBINE_TOKENS)), dim3(256), 0, s, partial,
                       zy, n_tokens, in.n_dev, in.rows, row_mask, n_tokens, p.n_splits, p.n_pad, inv_temperature, c, logprob,
                       entropy, lse, keep.buf ? keep.xref : static_cast<const float*>(nullptr),
                       keep.buf ? keep.unsafe : static_cast<uint8_t*>(nullptr));
}

// The forward that also prepares d_hidden.  With x = z c in the log2 domain and a per-token
// reference exponent ref_n (the scaled logit of the token's own label),
//   d_hidden[n] = sum_v dZ[n, v] W[v]
//               = s_n sum_{v != y} 2^(x_nv - ref_n) W[v] - g_n inv_T expm1(logprob_n) W[y_n],
//   s_n = -g_n inv_T 2^(ref_n - lse2_n),
// and the sum does not depend on the upstream gradient: it is accumulated while the logits exist,
// one vocabulary chunk at a time (the exponentials of the chunk as bf16 in a chunk-sized buffer,
// with the label's own entry left out; then wsum (+)= E_chunk * W_chunk in fp32).  A backward pass
// that only needs d_hidden is then one pass over [tokens, hidden]: 4 N H V matrix work for forward +
// backward instead of 6 N H V, and nothing is recomputed.  Tokens whose largest logit is too far
// above their label's are flagged in `unsafe`; their sums are not used (the backward recomputes them).
void enqueue_fwd_wsum(const FwdPlan& p, char* ws, const RowInputs& in, const uint8_t* row_mask, const void* weight,
                      int64_t n_tokens, int64_t hidden_dim, int64_t vocab, float inv_temperature, float* logprob,
                      float* entropy, float* lse, float* wsum, float* xref, uint8_t* unsafe, hipStream_t s) {
    float4* partial = reinterpret_cast<float4*>(ws + p.off_partial);
    float* zy = reinterpret_cast<float*>(ws + p.off_zy);
    uint32_t* queues = reinterpret_cast<uint32_t*>(ws + p.off_queue);
    uint16_t* chunk_buf = reinterpret_cast<uint16_t*>(ws + p.off_chunk);
    const float c = inv_temperature * OI_LOG2E;
    const uint16_t* Wp = static_cast<const uint16_t*>(weight);
    const int64_t h_tiles = (hidden_dim + BN - 1) / BN;
    const int64_t v_pad = p.vocab_tiles * BM;
    const int64_t splits_per_chunk = (p.chunk / BM + p.tiles_per_split - 1) / p.tiles_per_split;
    launch_label_ref(in, weight, n_tokens, hidden_dim, vocab, inv_temperature, xref, s);
    for (int64_t ci = 0; ci < p.n_chunks; ++ci) {
        const int64_t v_begin = ci * p.chunk;
        const int64_t v_end = v_begin + p.chunk < v_pad ? v_begin + p.chunk : v_pad;
        const int64_t cols = v_end - v_begin;                                   // multiple of 256
        const int64_t valid = vocab - v_begin < cols ? vocab - v_begin : cols;  // real rows of W
        const int64_t first = ci * splits_per_chunk;
        const int64_t n_first = p.n_splits - first < splits_per_chunk ? p.n_splits - first : splits_per_chunk;
        uint32_t* q = queues + ci * (FWD_QUEUE_WORDS + QUEUE_WORDS);
        const FwdLaunch fl = {p.tiles_per_split, p.long_splits, first, n_first, 0, chunk_buf, cols, v_begin / BM,
                              cols / BM, 1, xref};
        hipLaunchKernelGGL(lmhead_fwd_kernel<true>, dim3(resident_grid(n_first, p.token_tiles)), dim3(NTHREADS), 0, s, Wp,
                           in.hidden, in.labels, n_tokens, in.n_dev, hidden_dim, vocab, c, fl, p.n_pad, partial, zy, q);
        const Operand a = {chunk_buf, cols, 0, p.n_pad, cols};
        const Operand b = {Wp + v_begin * hidden_dim, hidden_dim, 0, hidden_dim, valid};
        const DynRows dyn = {in.n_dev, 1, nullptr, nullptr, nullptr, nullptr};
        hipLaunchKernelGGL((gemm_store_kernel<false, true>), dim3(resident_grid(p.n_pad / BM, h_tiles)), dim3(NTHREADS), 0,
                           s, a, p.n_pad, b, hidden_dim, round_up(valid, BK), ci == 0 ? 0 : 1, wsum,
                           static_cast<uint16_t*>(nullptr), hidden_dim, n_tokens, dyn, q + FWD_QUEUE_WORDS);
    }
    hipLaunchKernelGGL(lmhead_fwd_combine_kernel, dim3((unsigned)((n_tokens + COMBINE_TOKENS - 1) / COMBINE_TOKENS)), dim3(256), 0, s, partial,
                       zy, n_tokens, in.n_dev, in.rows, row_mask, n_tokens, p.n_splits, p.n_pad, inv_temperature, c, logprob,
                       entropy, lse, static_cast<const float*>(xref), unsafe);
}

// d_hidden row of selected token j (caller row rows[j], or j without a selection) from the weighted
// sum that the forward left behind; one workgroup per selected row.  The factor s is applied in two
// halves so that neither leaves the fp32 range.  Rows flagged in `unsafe` are left alone (the
// recomputing backward writes them).
__global__ void __launch_bounds__(256)
    dh_from_wsum_kernel(const float* __restrict__ wsum, const float* __restrict__ xref,
                        const uint8_t* __restrict__ unsafe, const uint16_t* __restrict__ W,
                        const int64_t* __restrict__ labels, const float* __restrict__ lse,
                        const float* __restrict__ logprob, const float* __restrict__ grad,
                        const int32_t* __restrict__ rows, const int32_t* __restrict__ count, int64_t n_tokens,
                        int64_t hdim, int64_t vocab, float inv_t, uint16_t* __restrict__ d_hidden) {
    const int64_t j = blockIdx.x;
    if (j >= (count ? (int64_t)*count : n_tokens)) return;
    const int64_t n = rows ? (int64_t)rows[j] : j;
    if (unsafe[n]) return;
    const float g = grad[n] * inv_t;
    const float half = __builtin_amdgcn_exp2f(0.5f * (xref[j] - lse[n] * OI_LOG2E));
    const float sb = -g * half;
    const float tl = -g * expm1f(logprob[n]);
    int64_t y = labels[n];
    y = y < 0 ? 0 : (y >= vocab ? vocab - 1 : y);
    const float4* src = reinterpret_cast<const float4*>(wsum + j * hdim);
    const uint2* wy = reinterpret_cast<const uint2*>(W + y * hdim);
    uint2* dst = reinterpret_cast<uint2*>(d_hidden + n * hdim);
    for (int64_t c = threadIdx.x; c < hdim / 4; c += blockDim.x) {  // hdim is a multiple of 64
        const float4 o = src[c];
        const uint2 w = wy[c];
        const float r0 = o.x * half * sb + tl * oi_bf16lo_to_f32(w.x), r1 = o.y * half * sb + tl * oi_bf16hi_to_f32(w.x);
        const float r2 = o.z * half * sb + tl * oi_bf16lo_to_f32(w.y), r3 = o.w * half * sb + tl * oi_bf16hi_to_f32(w.y);
        dst[c] = make_uint2(oi_pack_bf16x2(r0, r1), oi_pack_bf16x2(r2, r3));
    }
}

// The recomputing backward.  Per vocabulary chunk: dZ [n_pad, cols] (token-major, bf16, zero in padded
// rows and columns), then both products straight from W and the (selected) hidden rows, which enter
// as k-major operands:
//   d_hidden[n, h] (+)= sum_v dZ[n, v] * W[v_begin + v, h]      A k-contiguous, B k-major
//   d_weight[v_begin + v, h] = sum_n dZ[n, v] * hidden[n, h]    A k-major,      B k-major
// The sums stop at the last real vocabulary row / token (rounded up to a k-tile, whose missing
// rows are read from the last real one and meet zeros of dZ).  The queue words must be zeroed.
// dw_mode / dw32: how d_weight is stored.  2 (default): this call holds every token, bf16 rows are
// written directly.  0 / 1: the tokens come in several calls; dw32 (fp32 [vocab, hidden]) takes the
// first call's product (0) and adds the following ones (1; a call without tokens adds nothing and
// costs nothing); the caller rounds dw32 to bf16 when the last call is through.  4: the product is
// added to bf16 rows that an earlier call wrote.
// max_grid > 0 caps the number of resident workgroups of every launch (the queues work with any
// number): the launches that serve flagged rows normally find none, and a launch over a few CUs that
// finds nothing costs a fraction of one over all of them.
constexpr unsigned REPAIR_GRID = 32;
void enqueue_bwd(const BwdPlan& p, char* ws, const RowInputs& in, const void* weight, int64_t n_tokens,
                 int64_t hidden_dim, int64_t vocab, float inv_temperature, void* d_hidden, void* d_weight,
                 hipStream_t s, int dw_mode = 2, float* dw32 = nullptr, unsigned max_grid = 0) {
    auto grid_of = [&](int64_t tiles_m, int64_t tiles_n) {
        const unsigned g = resident_grid(tiles_m, tiles_n);
        return dim3(max_grid > 0 && g > max_grid ? max_grid : g);
    };
    uint16_t* dz = reinterpret_cast<uint16_t*>(ws + p.off_dz);
    float* dh32 = reinterpret_cast<float*>(ws + p.off_dh32);
    uint32_t* queues = reinterpret_cast<uint32_t*>(ws + p.off_queues);
    const uint16_t* Wp = static_cast<const uint16_t*>(weight);
    const float c = inv_temperature * OI_LOG2E;
    const int64_t h_tiles = (hidden_dim + BN - 1) / BN;
    for (int64_t ci = 0; ci < p.n_chunks; ++ci) {
        const int64_t v_begin = ci * p.chunk;
        const int64_t v_end = (ci + 1) * p.chunk < p.v_pad ? (ci + 1) * p.chunk : p.v_pad;
        const int64_t cols = v_end - v_begin;                                   // multiple of 256
        const int64_t valid = vocab - v_begin < cols ? vocab - v_begin : cols;  // real rows of W
        uint32_t* q = queues + ci * 3 * QUEUE_WORDS;
        hipLaunchKernelGGL(lmhead_dz_kernel, grid_of(cols / BM, p.n_pad / BN), dim3(NTHREADS), 0, s, Wp,
                           in.hidden, in.labels, in.lse, in.grad, in.logprob, n_tokens, in.n_dev, hidden_dim, vocab, c,
                           inv_temperature, v_begin, cols, p.n_pad, dz, q);
        const bool first = ci == 0, last = ci == p.n_chunks - 1;
        const int mode = last ? (first ? 2 : 3) : (first ? 0 : 1);
        {
            const Operand a = {dz, cols, 0, p.n_pad, cols};
            const Operand b = {Wp + v_begin * hidden_dim, hidden_dim, 0, hidden_dim, valid};
            const DynRows dyn = {in.n_dev, 1, in.rows, nullptr, nullptr, nullptr};
            hipLaunchKernelGGL((gemm_store_kernel<false, true>), grid_of(p.n_pad / BM, h_tiles),
                               dim3(NTHREADS), 0, s, a, p.n_pad, b, hidden_dim, round_up(valid, BK), mode, dh32,
                               static_cast<uint16_t*>(d_hidden), hidden_dim, n_tokens, dyn, q + QUEUE_WORDS);
        }
        if (d_weight) {
            const Operand a = {dz, cols, 0, cols, p.n_pad};
            const Operand b = {in.hidden, hidden_dim, 0, hidden_dim, n_tokens};
            const DynRows dyn = {in.n_dev, 2, nullptr, nullptr, nullptr, nullptr};
            hipLaunchKernelGGL((gemm_store_kernel<true, true>), grid_of(cols / BM, h_tiles),
                               dim3(NTHREADS), 0, s, a, cols, b, hidden_dim, round_up(n_tokens, BK), dw_mode,
                               dw32 ? dw32 + v_begin * hidden_dim : static_cast<float*>(nullptr),
                               static_cast<uint16_t*>(d_weight) + v_begin * hidden_dim, hidden_dim, valid, dyn,
                               q + 2 * QUEUE_WORDS);
        }
    }
}

// Both backward products of a slab from its kept exponentials (see slab_prepare_kernel): the whole
// vocabulary as one chunk, d_hidden rows stored once through the slab's row numbers, d_weight
// stored / accumulated as *dw_mode_dev says (the slab's place among the slabs of the call is known
// on the device only: the first one stores, the last one rounds to bf16, see SlabMeta).
// `queues`: 2 * QUEUE_WORDS zeroed words.
void enqueue_products_from_exponentials(const uint16_t* ecache, int64_t cache_ld, int64_t slab_pad,
                                        const int32_t* count, const int32_t* rows_s, const float* scale_a,
                                        const float* scale_b, const uint16_t* scaled_hidden, const void* weight,
                                        int64_t hidden_dim, int64_t vocab, void* d_hidden, void* d_weight,
                                        const int32_t* dw_mode_dev, float* dw32, uint32_t* queues, hipStream_t s) {
    const uint16_t* Wp = static_cast<const uint16_t*>(weight);
    const int64_t h_tiles = (hidden_dim + BN - 1) / BN;
    {
        const ProbeScope probe(1, s);
        const Operand a = {ecache, cache_ld, 0, slab_pad, cache_ld};
        const Operand b = {Wp, hidden_dim, 0, hidden_dim, vocab};
        const DynRows dyn = {count, 1, rows_s, scale_a, scale_b, nullptr};
        hipLaunchKernelGGL((gemm_store_kernel<false, true>), dim3(resident_grid(slab_pad / BM, h_tiles)),
                           dim3(NTHREADS), 0, s, a, slab_pad, b, hidden_dim, round_up(vocab, BK), 2,
                           static_cast<float*>(nullptr), static_cast<uint16_t*>(d_hidden), hidden_dim, slab_pad, dyn,
                           queues);
    }
    if (d_weight) {
        const ProbeScope probe(2, s);
        const Operand a = {ecache, cache_ld, 0, cache_ld, slab_pad};
        const Operand b = {scaled_hidden, hidden_dim, 0, hidden_dim, slab_pad};
        const DynRows dyn = {count, 2, nullptr, nullptr, nullptr, dw_mode_dev};
        hipLaunchKernelGGL((gemm_store_kernel<true, true>), dim3(resident_grid(cache_ld / BM, h_tiles)),
                           dim3(NTHREADS), 0, s, a, cache_ld, b, hidden_dim, round_up(slab_pad, BK), 2, dw32,
                           static_cast<uint16_t*>(d_weight), hidden_dim, vocab, dyn, queues + QUEUE_WORDS);
    }
}

// workspace of the whole-step entry point: forward and backward regions side by side (they share
// one row selection), the statistics partials, and the per-token vectors that connect the stages
struct StepPlan {
    FwdPlan fwd;
    BwdPlan bwd;
    size_t off_fwd, off_bwd, off_stats, off_lse, off_grad, off_denoms, total;
};
StepPlan plan_step(int64_t rows, int64_t cols, int64_t hdim, int64_t vocab) {
    StepPlan p;
    const int64_t n = rows * cols;
    p.fwd = plan_fwd(n, hdim, vocab, false);
    p.bwd = plan_bwd(n, hdim, vocab, true);
    Carver cv;
    p.off_fwd = cv.take(p.fwd.total);
    p.off_bwd = cv.take(p.bwd.total);
    p.off_stats = cv.take(oi_grpo_fused_workspace_bytes(rows, cols));
    p.off_lse = cv.take((size_t)n * sizeof(float));
    p.off_grad = cv.take((size_t)n * sizeof(float));
    p.off_denoms = cv.take((size_t)rows * sizeof(float));
    p.total = cv.off;
    return p;
}

// ---------------------------------------------------------------------------------------------
// The whole step in slabs of tokens, with nothing recomputed
// ---------------------------------------------------------------------------------------------
// The selected rows are taken a slab at a time (at most `cap` rows; the slabs of a call are made
// equal on the device, where the selected count lives).  A slab's forward leaves its exponentials
// (every vocabulary column, bf16, relative to each token's own reference exponent) in a slab-sized
// buffer, the slab's tokens get their upstream gradient at once (the caller of run_slab_passes says
// how: for the GRPO loss it depends only on the token's own logprob and on denominators that come
// from the mask), and both products read the buffer before the next slab overwrites it: d_hidden
// rows are final, d_weight accumulates in fp32 over the slabs.  6 N H V of matrix work instead of
// 8 N H V; the buffer holds [slab, vocabulary], never [tokens, vocabulary].  Tokens that the
// forward flags (largest logit too far above the label's) add nothing in their slab and are served
// by one recomputing backward over the flagged rows after the last slab, so the results do not
// depend on the size of the logits.  Every slab costs a pass over the fp32 d_weight and leaves the
// ends of its launches ragged.
constexpr int64_t SLAB_UNIT = 256;  // a slab capacity is a multiple of this many rows (a token tile)
constexpr int SLAB_QUEUE_WORDS = FWD_QUEUE_WORDS + 2 * QUEUE_WORDS;
struct SlabPlan {
    int64_t cap, n_passes, n_pad, v_pad;
    FwdPlan fwd;     // of one slab
    BwdPlan repair;  // the recomputing backward over all rows (for the flagged ones)
    size_t off_fwd, off_order, off_count, off_meta, off_unsafe, off_keep, off_repair, off_hidden_s, off_labels_s,
        off_rows_s, off_xref_s, off_scale_a, off_scale_b, off_scaled_hidden, off_queues, off_dw32, off_stats, off_lse,
        off_grad, off_denoms, total;
};
SlabPlan plan_slabs(int64_t n, int64_t stats_rows, int64_t stats_cols, int64_t hdim, int64_t vocab, bool want_dw,
                    int64_t slab_tokens, int64_t n_passes_override = 0) {
    SlabPlan p;
    p.n_pad = round_up(n, 256);
    p.v_pad = round_up(vocab, 256);
    const int64_t cap = round_up(slab_tokens < SLAB_UNIT ? SLAB_UNIT : slab_tokens, SLAB_UNIT);
    p.cap = p.n_pad < cap ? p.n_pad : cap;
    p.n_passes = n_passes_override > 0 ? n_passes_override : (p.n_pad + p.cap - 1) / p.cap;
    p.fwd = plan_fwd(p.cap, hdim, vocab, false);
    p.repair = plan_bwd(n, hdim, vocab, true);
    Carver cv;
    p.off_fwd = cv.take(p.fwd.total);
    p.off_order = cv.take((size_t)p.n_pad * sizeof(int32_t));
    p.off_count = cv.take(sizeof(int32_t));
    p.off_meta = cv.take((size_t)p.n_passes * sizeof(SlabMeta));
    p.off_unsafe = cv.take((size_t)p.n_pad);
    // the slab's exponentials and, after the last slab, the workspace of the repair share one region
    const size_t keep_bytes = (size_t)p.cap * p.v_pad * 2;
    p.off_keep = p.off_repair = cv.take(keep_bytes > p.repair.total ? keep_bytes : p.repair.total);
    p.off_hidden_s = cv.take((size_t)p.cap * hdim * 2);
    p.off_labels_s = cv.take((size_t)p.cap * sizeof(int64_t));
    p.off_rows_s = cv.take((size_t)p.cap * sizeof(int32_t));
    p.off_xref_s = cv.take((size_t)p.cap * sizeof(float));
    p.off_scale_a = cv.take((size_t)p.cap * sizeof(float));
    p.off_scale_b = cv.take((size_t)p.cap * sizeof(float));
    p.off_scaled_hidden = cv.take(want_dw ? (size_t)p.cap * hdim * 2 : 0);
    p.off_queues = cv.take((size_t)SLAB_QUEUE_WORDS * sizeof(uint32_t));
    p.off_dw32 = cv.take(want_dw && p.n_passes > 1 ? (size_t)vocab * hdim * sizeof(float) : 0);
    p.off_stats = cv.take(oi_grpo_fused_workspace_bytes(stats_rows, stats_cols));
    p.off_lse = cv.take((size_t)n * sizeof(float));
    p.off_grad = cv.take((size_t)n * sizeof(float));
    p.off_denoms = cv.take((size_t)stats_rows * sizeof(float));
    p.total = cv.off;
    return p;
}

// The selected rows split into the fewest slabs of at most `cap` rows: all of the same size (a multiple of
// 256 rows, the last one takes what is left), or, when that takes fewer rounds of tiles, full slabs of
// `cap` rows and a last one with the remainder.  What is counted is the slab's d_hidden product, the one
// tile kernel whose work items are long (a tile runs over the whole vocabulary): it has
// ceil(rows / 256) * h_tiles tiles for `grid` resident workgroups, and a round of tiles takes the same
// time whether it is full or not.  Passes past the last slab are empty.
__global__ void plan_slabs_kernel(const int32_t* __restrict__ count, int cap, int n_passes, int h_tiles, int grid,
                                  SlabMeta* __restrict__ meta) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_passes) return;
    const int n = *count;
    const int k = n > 0 ? (n + cap - 1) / cap : 1;
    int equal = ((n + k - 1) / k + 255) / 256 * 256;
    equal = equal > cap ? cap : equal;
    auto rounds = [&](int size) {
        int total = 0;
        for (int j = 0; j < k; ++j) {
            const int left = n - j * size;
            const int rows = left < 0 ? 0 : (left > size ? size : left);
            total += ((rows + 255) / 256 * h_tiles + grid - 1) / grid;
        }
        return total;
    };
    const int size = rounds(cap) < rounds(equal) ? cap : equal;
    const int left = n - i * size;
    meta[i].offset = i * size;
    meta[i].count = left < 0 ? 0 : (left > size ? size : left);
    const bool first = i == 0, last = i == k - 1;
    meta[i].dw_mode = i >= k ? -1 : (last ? (first ? 2 : 3) : (first ? 0 : 1));
    meta[i].reserved = 0;
}

// The per-token outputs start at zero: rows that take no part stay there, and the passes that look
// at every row before its own slab has run (the upstream gradient of a slab is computed for all rows)
// read zeros rather than whatever the caller's buffers held.
__global__ void zero_f32_kernel(int64_t n, float* __restrict__ a, float* __restrict__ b, float* __restrict__ c) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    a[i] = 0.f;
    if (b) b[i] = 0.f;
    if (c) c[i] = 0.f;
}

// What a slab-wise step is made of besides the passes themselves
struct SlabStep {
    const void *hidden, *weight;
    const int64_t* labels;       // per caller row, as the kernels score them
    const uint8_t* mask;         // per caller row: the rows that are multiplied
    int64_t n_tokens, hidden_dim, vocab;
    float inv_temperature;
    float *logprob, *entropy;    // per caller row (entropy may be null)
    void *d_hidden, *d_weight;   // d_weight may be null
};

// Runs the slab passes of `st` over the row index order[0 .. *count) that `plan_rows` leaves in the
// workspace together with the passes' SlabMeta.  `upstream(final)` must enqueue kernels that leave
// every caller row's d loss / d logprob in the workspace's grad vector, given the logprobs computed
// so far (the rows of the slabs up to the current one; with `final` set, all rows).
template <class PlanRows, class Upstream>
int run_slab_passes(const SlabPlan& p, char* ws, const SlabStep& st, hipStream_t s, PlanRows&& plan_rows,
                    Upstream&& upstream) {
    const int64_t n = st.n_tokens, hdim = st.hidden_dim, vocab = st.vocab;
    char* ws_fwd = ws + p.off_fwd;
    int32_t* order = reinterpret_cast<int32_t*>(ws + p.off_order);
    int32_t* count = reinterpret_cast<int32_t*>(ws + p.off_count);
    SlabMeta* meta = reinterpret_cast<SlabMeta*>(ws + p.off_meta);
    uint8_t* unsafe = reinterpret_cast<uint8_t*>(ws + p.off_unsafe);
    uint16_t* keep_buf = reinterpret_cast<uint16_t*>(ws + p.off_keep);
    uint16_t* hidden_s = reinterpret_cast<uint16_t*>(ws + p.off_hidden_s);
    int64_t* labels_s = reinterpret_cast<int64_t*>(ws + p.off_labels_s);
    int32_t* rows_s = reinterpret_cast<int32_t*>(ws + p.off_rows_s);
    float* xref_s = reinterpret_cast<float*>(ws + p.off_xref_s);
    float* scale_a = reinterpret_cast<float*>(ws + p.off_scale_a);
    float* scale_b = reinterpret_cast<float*>(ws + p.off_scale_b);
    uint16_t* scaled_hidden = st.d_weight ? reinterpret_cast<uint16_t*>(ws + p.off_scaled_hidden) : nullptr;
    uint32_t* queues = reinterpret_cast<uint32_t*>(ws + p.off_queues);
    float* dw32 = st.d_weight && p.n_passes > 1 ? reinterpret_cast<float*>(ws + p.off_dw32) : nullptr;
    float* lse = reinterpret_cast<float*>(ws + p.off_lse);
    float* grad = reinterpret_cast<float*>(ws + p.off_grad);
    const uint16_t* hid = static_cast<const uint16_t*>(st.hidden);

    hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((p.n_pad / 4 + 255) / 256)), dim3(256), 0, s,
                       reinterpret_cast<uint32_t*>(unsafe), (int)(p.n_pad / 4));
    plan_rows(order, count, meta);
    hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, st.logprob, st.entropy, lse);
    hipLaunchKernelGGL(zero_unselected_rows_kernel, dim3((unsigned)n), dim3(256), 0, s, st.mask,
                       static_cast<const float*>(nullptr), hdim, static_cast<uint16_t*>(st.d_hidden));
    for (int64_t i = 0; i < p.n_passes; ++i) {
        const int32_t* cnt = &meta[i].count;
        hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, s, queues, SLAB_QUEUE_WORDS);
        hipLaunchKernelGGL(gather_slab_kernel, dim3((unsigned)p.cap), dim3(256), 0, s, hid, st.labels,
                           static_cast<const float*>(nullptr), static_cast<const float*>(nullptr),
                           static_cast<const float*>(nullptr), order, meta + i, hdim, hidden_s, labels_s, rows_s,
                           static_cast<float*>(nullptr), static_cast<float*>(nullptr), static_cast<float*>(nullptr));
        const RowInputs in = {hidden_s, labels_s, nullptr, nullptr, rows_s, cnt, nullptr};
        launch_label_ref(in, st.weight, p.cap, hdim, vocab, st.inv_temperature, xref_s, s);
        const KeepPlan keep = {keep_buf, p.v_pad, p.v_pad / BM, xref_s, unsafe};
        // the forward's own queue words are the first FWD_QUEUE_WORDS of `queues`
        FwdPlan fp = p.fwd;
        fp.off_queue = (size_t)(reinterpret_cast<char*>(queues) - ws_fwd);
        enqueue_fwd(fp, ws_fwd, in, nullptr, st.weight, p.cap, hdim, vocab, st.inv_temperature, st.logprob, st.entropy,
                    lse, keep, s);
        const int rc = upstream(false);
        if (rc != OI_OK) return rc;
        hipLaunchKernelGGL(slab_prepare_kernel, dim3((unsigned)p.cap), dim3(256), 0, s, lse, grad, st.logprob, unsafe,
                           rows_s, labels_s, xref_s, meta + i, st.inv_temperature, vocab, hdim, keep_buf, p.v_pad,
                           hidden_s, scale_a, scale_b, scaled_hidden);
        enqueue_products_from_exponentials(keep_buf, p.v_pad, p.cap, cnt, rows_s, scale_a, scale_b, scaled_hidden,
                                           st.weight, hdim, vocab, st.d_hidden, st.d_weight, &meta[i].dw_mode, dw32,
                                           queues + FWD_QUEUE_WORDS, s);
    }
    // the flagged rows, if any: one recomputing backward over them (its workspace takes the place of
    // the exponentials), added to what the slabs left in d_weight
    {
        const int rc = upstream(true);
        if (rc != OI_OK) return rc;
        char* ws_rep = ws + p.off_repair;
        uint32_t* rq = reinterpret_cast<uint32_t*>(ws_rep + p.repair.off_queues);
        const int n_words = (int)(3 * p.repair.n_chunks * QUEUE_WORDS);
        const bool select_clears = n_words <= SELECT_THREADS;
        if (!select_clears)
            hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((n_words + 255) / 256)), dim3(256), 0, s, rq, n_words);
        const RowInputs in = launch_selection(p.repair.sel, ws_rep, st.hidden, st.labels, lse, grad, unsafe, false, n,
                                              hdim, rq, select_clears ? n_words : 0, s, st.logprob);
        enqueue_bwd(p.repair, ws_rep, in, st.weight, n, hdim, vocab, st.inv_temperature, st.d_hidden, st.d_weight, s, 4,
                    nullptr, REPAIR_GRID);
    }
    return oi_launch_status();
}

}  // namespace

extern "C" size_t oi_lmhead_fwd_workspace_bytes(int64_t n_tokens, int64_t hidden_dim, int64_t vocab,
                                                int with_row_mask) {
    if (n_tokens <= 0 || vocab <= 0 || hidden_dim <= 0) return 0;
    return plan_fwd(n_tokens, hidden_dim, vocab, with_row_mask != 0).total;
}

extern "C" int oi_lmhead_logp_fwd(const void* hidden, const void* weight, const int64_t* labels,
                                  const uint8_t* row_mask, int64_t n_tokens, int64_t hidden_dim, int64_t vocab,
                                  float inv_temperature, float* logprob, float* entropy, float* lse, void* workspace,
                                  size_t workspace_bytes, void* stream) {
    int rc = check_lmhead(hidden, weight, labels, n_tokens, hidden_dim, vocab, inv_temperature);
    if (rc != OI_OK) return rc;
    if (n_tokens == 0) return OI_OK;
    OI_RETURN_IF(!logprob || !workspace, OI_ENULL);
    OI_RETURN_IF(!oi_aligned(workspace, 256), OI_EALIGN);
    const FwdPlan p = plan_fwd(n_tokens, hidden_dim, vocab, row_mask != nullptr);
    OI_RETURN_IF(workspace_bytes < p.total, OI_EWORKSPACE);
    char* ws = static_cast<char*>(workspace);
    uint32_t* queue = reinterpret_cast<uint32_t*>(ws + p.off_queue);
    hipStream_t s = static_cast<hipStream_t>(stream);
    RowInputs in = {static_cast<const uint16_t*>(hidden), labels, nullptr, nullptr, nullptr, nullptr, nullptr};
    if (row_mask)
        in = launch_selection(p.sel, ws, hidden, labels, nullptr, nullptr, row_mask, false, n_tokens, hidden_dim, queue,
                              FWD_QUEUE_WORDS, s);
    else
        hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, s, queue, FWD_QUEUE_WORDS);
    enqueue_fwd(p, ws, in, row_mask, weight, n_tokens, hidden_dim, vocab, inv_temperature, logprob, entropy, lse,
                KeepPlan{nullptr, 0, 0, nullptr, nullptr}, s);
    return oi_launch_status();
}

extern "C" size_t oi_lmhead_fwd_wsum_workspace_bytes(int64_t n_tokens, int64_t hidden_dim, int64_t vocab,
                                                     int with_row_mask) {
    if (n_tokens <= 0 || vocab <= 0 || hidden_dim <= 0) return 0;
    return plan_fwd(n_tokens, hidden_dim, vocab, with_row_mask != 0, true).total;
}

extern "C" int oi_lmhead_logp_fwd_wsum(const void* hidden, const void* weight, const int64_t* labels,
                                       const uint8_t* row_mask, int64_t n_tokens, int64_t hidden_dim, int64_t vocab,
                                       float inv_temperature, float* logprob, float* entropy, float* lse, float* wsum,
                                       float* xref, uint8_t* unsafe, void* workspace, size_t workspace_bytes,
                                       void* stream) {
    int rc = check_lmhead(hidden, weight, labels, n_tokens, hidden_dim, vocab, inv_temperature);
    if (rc != OI_OK) return rc;
    if (n_tokens == 0) return OI_OK;
    OI_RETURN_IF(!logprob || !lse || !wsum || !xref || !unsafe || !workspace, OI_ENULL);
    OI_RETURN_IF(!oi_aligned(workspace, 256) || !oi_aligned(wsum, 16) || !oi_aligned(xref, 4), OI_EALIGN);
    const FwdPlan p = plan_fwd(n_tokens, hidden_dim, vocab, row_mask != nullptr, true);
    OI_RETURN_IF(workspace_bytes < p.total, OI_EWORKSPACE);
    char* ws = static_cast<char*>(workspace);
    uint32_t* queues = reinterpret_cast<uint32_t*>(ws + p.off_queue);
    const int n_queue_words = (int)(p.n_chunks * (FWD_QUEUE_WORDS + QUEUE_WORDS));
    hipStream_t s = static_cast<hipStream_t>(stream);
    RowInputs in = {static_cast<const uint16_t*>(hidden), labels, nullptr, nullptr, nullptr, nullptr, nullptr};
    const bool select_clears_queues = row_mask && n_queue_words <= SELECT_THREADS;
    if (!select_clears_queues)
        hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((n_queue_words + 255) / 256)), dim3(256), 0, s, queues,
                           n_queue_words);
    if (row_mask)
        in = launch_selection(p.sel, ws, hidden, labels, nullptr, nullptr, row_mask, false, n_tokens, hidden_dim, queues,
                              select_clears_queues ? n_queue_words : 0, s);
    hipLaunchKernelGGL(zero_bytes_kernel, dim3((unsigned)((n_tokens + 255) / 256)), dim3(256), 0, s, unsafe, n_tokens);
    enqueue_fwd_wsum(p, ws, in, row_mask, weight, n_tokens, hidden_dim, vocab, inv_temperature, logprob, entropy, lse,
                     wsum, xref, unsafe, s);
    return oi_launch_status();
}

namespace {
// workspace of oi_lmhead_dh_from_wsum: the row index of the mask, and the recomputing backward for
// the rows that the forward flagged
struct DhPlan {
    BwdPlan repair;
    size_t off_rows, off_count, off_repair, total;
};
DhPlan plan_dh(int64_t n_tokens, int64_t hdim, int64_t vocab) {
    DhPlan p;
    p.repair = plan_bwd(n_tokens, hdim, vocab, true);
    Carver cv;
    p.off_rows = cv.take((size_t)round_up(n_tokens, 256) * sizeof(int32_t));
    p.off_count = cv.take(sizeof(int32_t));
    p.off_repair = cv.take(p.repair.total);
    p.total = cv.off;
    return p;
}
}  // namespace

extern "C" size_t oi_lmhead_dh_workspace_bytes(int64_t n_tokens, int64_t hidden_dim, int64_t vocab) {
    if (n_tokens <= 0 || hidden_dim <= 0 || vocab <= 0) return 0;
    return plan_dh(n_tokens, hidden_dim, vocab).total;
}

extern "C" int oi_lmhead_dh_from_wsum(const void* hidden, const void* weight, const int64_t* labels, const float* lse,
                                      const float* logprob, const float* grad_logprob, const uint8_t* row_mask,
                                      const float* wsum, const float* xref, const uint8_t* unsafe, int64_t n_tokens,
                                      int64_t hidden_dim, int64_t vocab, float inv_temperature, void* d_hidden,
                                      void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_lmhead(hidden, weight, labels, n_tokens, hidden_dim, vocab, inv_temperature);
    if (rc != OI_OK) return rc;
    if (n_tokens == 0) return OI_OK;
    OI_RETURN_IF(!lse || !logprob || !grad_logprob || !wsum || !xref || !unsafe || !d_hidden || !workspace, OI_ENULL);
    OI_RETURN_IF(!oi_aligned(wsum, 16) || !oi_aligned(d_hidden, 8) || !oi_aligned(workspace, 256), OI_EALIGN);
    const DhPlan p = plan_dh(n_tokens, hidden_dim, vocab);
    OI_RETURN_IF(workspace_bytes < p.total, OI_EWORKSPACE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    char* ws = static_cast<char*>(workspace);
    const int32_t *rows = nullptr, *count = nullptr;
    if (row_mask) {
        // the same ascending selection as in the forward pass, rebuilt from the same mask
        int32_t* r = reinterpret_cast<int32_t*>(ws + p.off_rows);
        int32_t* c = reinterpret_cast<int32_t*>(ws + p.off_count);
        hipLaunchKernelGGL(select_rows_kernel, dim3(1), dim3(SELECT_THREADS), 0, s, row_mask,
                           static_cast<const float*>(nullptr), n_tokens, r, c, static_cast<uint32_t*>(nullptr), 0);
        hipLaunchKernelGGL(zero_unselected_rows_kernel, dim3((unsigned)n_tokens), dim3(256), 0, s, row_mask,
                           static_cast<const float*>(nullptr), hidden_dim, static_cast<uint16_t*>(d_hidden));
        rows = r;
        count = c;
    }
    hipLaunchKernelGGL(dh_from_wsum_kernel, dim3((unsigned)n_tokens), dim3(256), 0, s, wsum, xref, unsafe,
                       static_cast<const uint16_t*>(weight), labels, lse, logprob, grad_logprob, rows, count, n_tokens,
                       hidden_dim, vocab, inv_temperature, static_cast<uint16_t*>(d_hidden));
    // the flagged rows (a subset of the mask's), recomputed; normally none
    char* ws_rep = ws + p.off_repair;
    uint32_t* rq = reinterpret_cast<uint32_t*>(ws_rep + p.repair.off_queues);
    const int n_words = (int)(3 * p.repair.n_chunks * QUEUE_WORDS);
    const bool select_clears = n_words <= SELECT_THREADS;
    if (!select_clears)
        hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((n_words + 255) / 256)), dim3(256), 0, s, rq, n_words);
    const RowInputs in = launch_selection(p.repair.sel, ws_rep, hidden, labels, lse, grad_logprob, unsafe, false,
                                          n_tokens, hidden_dim, rq, select_clears ? n_words : 0, s, logprob);
    enqueue_bwd(p.repair, ws_rep, in, weight, n_tokens, hidden_dim, vocab, inv_temperature, d_hidden, nullptr, s, 2, nullptr,
                REPAIR_GRID);
    return oi_launch_status();
}

extern "C" size_t oi_lmhead_bwd_workspace_bytes(int64_t n_tokens, int64_t hidden_dim, int64_t vocab,
                                                int want_d_weight, int with_row_selection) {
    if (n_tokens <= 0 || hidden_dim <= 0 || vocab <= 0) return 0;
    (void)want_d_weight;
    return plan_bwd(n_tokens, hidden_dim, vocab, with_row_selection != 0).total;
}

extern "C" int oi_lmhead_logp_bwd(const void* hidden, const void* weight, const int64_t* labels, const float* lse,
                                  const float* grad_logprob, const uint8_t* row_mask, int skip_zero_grad_rows,
                                  int64_t n_tokens, int64_t hidden_dim, int64_t vocab, float inv_temperature,
                                  const float* logprob, void* d_hidden, void* d_weight, void* workspace,
                                  size_t workspace_bytes, void* stream) {
    int rc = check_lmhead(hidden, weight, labels, n_tokens, hidden_dim, vocab, inv_temperature);
    if (rc != OI_OK) return rc;
    if (n_tokens == 0) return OI_OK;
    OI_RETURN_IF(!lse || !grad_logprob || !logprob || !d_hidden || !workspace, OI_ENULL);
    // bf16 results are stored as pairs (4-byte words)
    OI_RETURN_IF(!oi_aligned(workspace, 256) || !oi_aligned(d_hidden, 4) || !oi_aligned(d_weight, 4), OI_EALIGN);
    const bool selecting = row_mask != nullptr || skip_zero_grad_rows != 0;
    const BwdPlan p = plan_bwd(n_tokens, hidden_dim, vocab, selecting);
    OI_RETURN_IF(workspace_bytes < p.total, OI_EWORKSPACE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    char* ws = static_cast<char*>(workspace);
    uint32_t* queues = reinterpret_cast<uint32_t*>(ws + p.off_queues);
    const int n_queue_words = (int)(3 * p.n_chunks * QUEUE_WORDS);
    const float* zero_grad_probe = skip_zero_grad_rows ? grad_logprob : nullptr;
    RowInputs in = {static_cast<const uint16_t*>(hidden), labels, lse, grad_logprob, nullptr, nullptr, logprob};
    const bool select_clears_queues = selecting && n_queue_words <= SELECT_THREADS;
    if (!select_clears_queues)
        hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((n_queue_words + 255) / 256)), dim3(256), 0, s, queues,
                           n_queue_words);
    if (selecting) {
        in = launch_selection(p.sel, ws, hidden, labels, lse, grad_logprob, row_mask, skip_zero_grad_rows != 0, n_tokens,
                              hidden_dim, queues, select_clears_queues ? n_queue_words : 0, s,
                              logprob);
        hipLaunchKernelGGL(zero_unselected_rows_kernel, dim3((unsigned)n_tokens), dim3(256), 0, s, row_mask,
                           zero_grad_probe, hidden_dim, static_cast<uint16_t*>(d_hidden));
    }
    enqueue_bwd(p, ws, in, weight, n_tokens, hidden_dim, vocab, inv_temperature, d_hidden, d_weight, s);
    return oi_launch_status();
}

extern "C" size_t oi_lmhead_grpo_workspace_bytes(int64_t rows, int64_t cols, int64_t hidden_dim, int64_t vocab,
                                                 int want_d_weight, int64_t slab_tokens) {
    if (rows <= 0 || cols <= 0 || hidden_dim <= 0 || vocab <= 0) return 0;
    if (slab_tokens > 0) return plan_slabs(rows * cols, rows, cols, hidden_dim, vocab, want_d_weight != 0, slab_tokens).total;
    return plan_step(rows, cols, hidden_dim, vocab).total;
}

namespace {
// oi_lmhead_grpo_fwd_bwd in slabs of tokens (slab_tokens > 0); arguments as checked by the entry point
int grpo_step_in_slabs(const void* hidden, const void* weight, const int64_t* labels, const uint8_t* mask,
                       const float* old_logprobs, const float* ref_logprobs, const float* advantages,
                       const float* rho_weights, int64_t rows, int64_t cols, int64_t hidden_dim, int64_t vocab,
                       float inv_temperature, int loss_fn, float ratio_lo, float ratio_hi, int kl_estimator, float beta,
                       int axis_mode, float denominator, float scale, float* logprob, float* entropy, float* out_stats,
                       void* d_hidden, void* d_weight, int64_t slab_tokens, void* workspace, size_t workspace_bytes,
                       void* stream) {
    const int64_t n_tokens = rows * cols;
    const SlabPlan p = plan_slabs(n_tokens, rows, cols, hidden_dim, vocab, d_weight != nullptr, slab_tokens);
    OI_RETURN_IF(workspace_bytes < p.total, OI_EWORKSPACE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    char* ws = static_cast<char*>(workspace);
    float* grad = reinterpret_cast<float*>(ws + p.off_grad);
    float* row_denoms = reinterpret_cast<float*>(ws + p.off_denoms);
    // the denominators come from the mask alone: a first pass of the statistics over logprobs that are
    // not there yet (zeros) leaves them in row_denoms (its other results are overwritten at the end)
    hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((n_tokens + 255) / 256)), dim3(256), 0, s, n_tokens, logprob, entropy,
                       static_cast<float*>(nullptr));
    int rc = oi_grpo_fused_fwd(logprob, old_logprobs, ref_logprobs, advantages, mask, rho_weights, entropy, nullptr, nullptr,
                               nullptr, nullptr, rows, cols, loss_fn, ratio_lo, ratio_hi, kl_estimator, beta, axis_mode,
                               denominator, scale, out_stats, row_denoms, ws + p.off_stats,
                               oi_grpo_fused_workspace_bytes(rows, cols), stream);
    if (rc != OI_OK) return rc;
    const SlabStep st = {hidden, weight, labels, mask, n_tokens, hidden_dim, vocab, inv_temperature, logprob, entropy,
                         d_hidden, d_weight};
    rc = run_slab_passes(
        p, ws, st, s,
        [&](int32_t* order, int32_t* count, SlabMeta* meta) {
            hipLaunchKernelGGL(select_rows_kernel, dim3(1), dim3(SELECT_THREADS), 0, s, mask,
                               static_cast<const float*>(nullptr), n_tokens, order, count,
                               static_cast<uint32_t*>(nullptr), 0);
            const int64_t h_tiles = (hidden_dim + BN - 1) / BN;
            hipLaunchKernelGGL(plan_slabs_kernel, dim3((unsigned)((p.n_passes + 63) / 64)), dim3(64), 0, s, count,
                               (int)p.cap, (int)p.n_passes, (int)h_tiles, (int)resident_grid(p.cap / BM, h_tiles), meta);
        },
        [&](bool) {
            // every token's d loss / d logprob from its own logprob; tokens of later slabs hold numbers
            // that nobody reads before their own slab has overwritten them
            return oi_grpo_fused_bwd(logprob, old_logprobs, ref_logprobs, advantages, mask, rho_weights, rows, cols,
                                     loss_fn, ratio_lo, ratio_hi, kl_estimator, beta, scale, row_denoms, nullptr, grad,
                                     stream);
        });
    if (rc != OI_OK) return rc;
    // loss and statistics from all logprobs
    return oi_grpo_fused_fwd(logprob, old_logprobs, ref_logprobs, advantages, mask, rho_weights, entropy, nullptr, nullptr,
                             nullptr, nullptr, rows, cols, loss_fn, ratio_lo, ratio_hi, kl_estimator, beta, axis_mode,
                             denominator, scale, out_stats, row_denoms, ws + p.off_stats,
                             oi_grpo_fused_workspace_bytes(rows, cols), stream);
}
}  // namespace

extern "C" int oi_lmhead_grpo_fwd_bwd(const void* hidden, const void* weight, const int64_t* labels,
                                      const uint8_t* mask, const float* old_logprobs, const float* ref_logprobs,
                                      const float* advantages, const float* rho_weights, int64_t rows, int64_t cols,
                                      int64_t hidden_dim, int64_t vocab, float inv_temperature, int loss_fn,
                                      float ratio_lo, float ratio_hi, int kl_estimator, float beta, int axis_mode,
                                      float denominator, float scale, float* logprob, float* entropy, float* out_stats,
                                      void* d_hidden, void* d_weight, int64_t slab_tokens, void* workspace,
                                      size_t workspace_bytes, void* stream) {
    OI_RETURN_IF(rows <= 0 || cols <= 0 || rows > MAX_LD || cols > MAX_LD || slab_tokens < 0, OI_EINVAL);
    const int64_t n_tokens = rows * cols;
    int rc = check_lmhead(hidden, weight, labels, n_tokens, hidden_dim, vocab, inv_temperature);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(!mask || !advantages || !logprob || !out_stats || !d_hidden || !workspace, OI_ENULL);
    OI_RETURN_IF(!oi_aligned(workspace, 256) || !oi_aligned(d_hidden, 4) || !oi_aligned(d_weight, 4), OI_EALIGN);
    if (slab_tokens > 0)
        return grpo_step_in_slabs(hidden, weight, labels, mask, old_logprobs, ref_logprobs, advantages, rho_weights, rows,
                                  cols, hidden_dim, vocab, inv_temperature, loss_fn, ratio_lo, ratio_hi, kl_estimator,
                                  beta, axis_mode, denominator, scale, logprob, entropy, out_stats, d_hidden, d_weight,
                                  slab_tokens, workspace, workspace_bytes, stream);
    const StepPlan p = plan_step(rows, cols, hidden_dim, vocab);
    OI_RETURN_IF(workspace_bytes < p.total, OI_EWORKSPACE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    char* ws = static_cast<char*>(workspace);
    char* ws_fwd = ws + p.off_fwd;
    char* ws_bwd = ws + p.off_bwd;
    float* lse = reinterpret_cast<float*>(ws + p.off_lse);
    float* grad = reinterpret_cast<float*>(ws + p.off_grad);
    float* row_denoms = reinterpret_cast<float*>(ws + p.off_denoms);

    // one selection for both passes: it lives in the backward region; the select kernel also clears
    // the backward queues, the forward queue gets the small fill kernel
    uint32_t* fwd_queue = reinterpret_cast<uint32_t*>(ws_fwd + p.fwd.off_queue);
    uint32_t* bwd_queues = reinterpret_cast<uint32_t*>(ws_bwd + p.bwd.off_queues);
    const int n_queue_words = (int)(3 * p.bwd.n_chunks * QUEUE_WORDS);
    const bool select_clears_queues = n_queue_words <= SELECT_THREADS;
    hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, s, fwd_queue, FWD_QUEUE_WORDS);
    if (!select_clears_queues)
        hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((n_queue_words + 255) / 256)), dim3(256), 0, s,
                           bwd_queues, n_queue_words);
    RowInputs in = launch_selection(p.bwd.sel, ws_bwd, hidden, labels, nullptr, nullptr, mask, false, n_tokens,
                                    hidden_dim, bwd_queues, select_clears_queues ? n_queue_words : 0, s);
    enqueue_fwd(p.fwd, ws_fwd, in, mask, weight, n_tokens, hidden_dim, vocab, inv_temperature, logprob, entropy, lse,
                KeepPlan{nullptr, 0, 0, nullptr, nullptr}, s);

    // loss and statistics from the logprobs, then every token's d loss / d logprob (upstream gradient 1)
    rc = oi_grpo_fused_fwd(logprob, old_logprobs, ref_logprobs, advantages, mask, rho_weights, entropy, nullptr, nullptr,
                           nullptr, nullptr, rows, cols, loss_fn, ratio_lo, ratio_hi, kl_estimator, beta, axis_mode,
                           denominator, scale, out_stats, row_denoms, ws + p.off_stats,
                           oi_grpo_fused_workspace_bytes(rows, cols), stream);
    if (rc != OI_OK) return rc;
    rc = oi_grpo_fused_bwd(logprob, old_logprobs, ref_logprobs, advantages, mask, rho_weights, rows, cols, loss_fn,
                           ratio_lo, ratio_hi, kl_estimator, beta, scale, row_denoms, nullptr, grad, stream);
    if (rc != OI_OK) return rc;

    float* lse_c = reinterpret_cast<float*>(ws_bwd + p.bwd.sel.off_lse);
    float* grad_c = reinterpret_cast<float*>(ws_bwd + p.bwd.sel.off_grad);
    float* logprob_c = reinterpret_cast<float*>(ws_bwd + p.bwd.sel.off_logprob);
    hipLaunchKernelGGL(gather_f32_kernel, dim3((unsigned)((n_tokens + 255) / 256)), dim3(256), 0, s, lse, grad, logprob,
                       in.rows, in.n_dev, lse_c, grad_c, logprob_c);
    in.lse = lse_c;
    in.grad = grad_c;
    in.logprob = logprob_c;
    hipLaunchKernelGGL(zero_unselected_rows_kernel, dim3((unsigned)n_tokens), dim3(256), 0, s, mask,
                       static_cast<const float*>(nullptr), hidden_dim, static_cast<uint16_t*>(d_hidden));
    enqueue_bwd(p.bwd, ws_bwd, in, weight, n_tokens, hidden_dim, vocab, inv_temperature, d_hidden, d_weight, s);
    return oi_launch_status();
}

// ---------------------------------------------------------------------------------------------
// The whole DPO step on hidden states, in slabs of whole chosen / rejected pairs
// ---------------------------------------------------------------------------------------------
namespace {
// Workgroup s handles sequence s: every position t of its range gets the label it is scored against
// (labels[t + 1]) and a mask byte (that label is not -100); the number of scored positions goes to
// cnt[s].  The positions that belong to no range (the last one of a padded row, of the packed row)
// are masked out.
__global__ void __launch_bounds__(256)
    dpo_rows_kernel(const int64_t* __restrict__ labels, const int32_t* __restrict__ cu, int64_t n_seqs, int64_t total,
                    int64_t* __restrict__ labels_eff, uint8_t* __restrict__ mask, int32_t* __restrict__ cnt) {
    const int64_t s = blockIdx.x;
    int64_t a, b;
    oi_seq_range(cu, s, n_seqs, total, &a, &b);
    float c = 0.f;
    for (int64_t t = a + threadIdx.x; t < b; t += blockDim.x) {
        const int64_t y = labels[t + 1];
        labels_eff[t] = y;
        const bool keep = y != -100;
        mask[t] = keep ? 1 : 0;
        c += keep ? 1.f : 0.f;
    }
    __shared__ float scratch[16];
    c = oi_block_sum(c, scratch);  // exact: at most 2^22 positions per sequence
    if (threadIdx.x == 0) {
        cnt[s] = (int32_t)c;
        const int64_t last = cu ? (s == n_seqs - 1 ? total - 1 : -1) : s * total + total - 1;
        if (last >= 0) {
            labels_eff[last] = -100;
            mask[last] = 0;
        }
    }
}

// One thread.  The scored rows are taken pair by pair (pair p = sequences p and n_seqs / 2 + p, the
// chosen and the rejected answer to one prompt: open_instruct/dpo_utils.py:734-763, 876-877): off[s]
// is where sequence s starts in the row index, and the slabs are filled with whole pairs in that order
// (a pair that does not fit the current slab starts the next one), because the upstream gradient of a
// token depends on the logprob sums of both sequences of its pair and must be known when the slab's
// exponentials are multiplied.  A pair with more rows than a slab holds is cut across slabs and its
// sequences are marked (seq_unsafe): their tokens take the recomputing backward after the last slab.
// Two consecutive slabs always hold more than `cap` rows together, so 2 ceil(rows / cap) + 1 passes
// are enough.
__global__ void dpo_plan_kernel(const int32_t* __restrict__ cnt, int n_seqs, int cap, int n_passes,
                                int32_t* __restrict__ off, uint8_t* __restrict__ seq_unsafe, int32_t* __restrict__ count,
                                SlabMeta* __restrict__ meta) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    const int bs = n_seqs / 2;
    int run = 0;
    for (int p = 0; p < bs; ++p) {
        off[p] = run;
        run += cnt[p];
        off[bs + p] = run;
        run += cnt[bs + p];
    }
    *count = run;
    int i = 0, start = 0, fill = 0;
    auto close = [&]() {
        if (i < n_passes) {
            meta[i].offset = start;
            meta[i].count = fill;
        }
        ++i;
        start += fill;
        fill = 0;
    };
    for (int p = 0; p < bs; ++p) {
        int rows = cnt[p] + cnt[bs + p];
        const bool oversize = rows > cap;
        seq_unsafe[p] = seq_unsafe[bs + p] = oversize ? 1 : 0;
        if (oversize) {
            while (rows > 0) {
                const int take = rows < cap - fill ? rows : cap - fill;
                fill += take;
                rows -= take;
                if (fill == cap) close();
            }
        } else {
            if (fill + rows > cap) close();
            fill += rows;
        }
    }
    if (fill > 0) close();
    const int k = i < n_passes ? i : n_passes;  // slabs with rows (at least the one that stores zeros)
    for (int j = k; j < n_passes; ++j) {
        meta[j].offset = start;
        meta[j].count = 0;
    }
    const int kk = k > 0 ? k : 1;
    for (int j = 0; j < n_passes; ++j) {
        const bool first = j == 0, last = j == kk - 1;
        meta[j].dw_mode = j >= kk ? -1 : (last ? (first ? 2 : 3) : (first ? 0 : 1));
        meta[j].reserved = 0;
    }
}

// Workgroup s writes the scored positions of sequence s, in ascending order, to
// order[off[s] .. off[s] + cnt[s]) and marks them in `unsafe` when the sequence is marked.
__global__ void __launch_bounds__(256)
    dpo_order_kernel(const uint8_t* __restrict__ mask, const int32_t* __restrict__ cu, int64_t n_seqs, int64_t total,
                     const int32_t* __restrict__ off, const uint8_t* __restrict__ seq_unsafe,
                     int32_t* __restrict__ order, uint8_t* __restrict__ unsafe) {
    const int64_t s = blockIdx.x;
    int64_t a, b;
    oi_seq_range(cu, s, n_seqs, total, &a, &b);
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int64_t per = (b - a + 255) / 256;
    const int64_t lo = a + t * per, hi = lo + per < b ? lo + per : b;
    int c = 0;
    for (int64_t i = lo; i < hi; ++i) c += mask[i] ? 1 : 0;
    int incl = c;
#pragma unroll
    for (int o = 1; o < OI_WAVE; o <<= 1) {
        const int up = __shfl_up(incl, o, OI_WAVE);
        if (lane >= o) incl += up;
    }
    __shared__ int wave_total[4];
    if (lane == OI_WAVE - 1) wave_total[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += wave_total[w];
    int pos = off[s] + base + incl - c;
    const bool flag = seq_unsafe[s] != 0;
    for (int64_t i = lo; i < hi; ++i)
        if (mask[i]) {
            order[pos++] = (int32_t)i;
            if (flag) unsafe[i] = 1;
        }
}

__global__ void fill_f32_kernel(float* __restrict__ p, int64_t n, float v) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

struct DpoPlan {
    SlabPlan slabs;
    int64_t n, bs;
    size_t off_slabs, off_labels_eff, off_mask, off_cnt, off_off, off_seq_unsafe, off_counts, off_dseq, off_gl, total;
};
DpoPlan plan_dpo(int64_t n_seqs, int64_t total, bool packed, int64_t hdim, int64_t vocab, bool want_dw,
                 int64_t slab_tokens) {
    DpoPlan p;
    p.n = packed ? total : n_seqs * total;
    p.bs = n_seqs / 2;
    const int64_t n_pad = round_up(p.n, 256);
    const int64_t cap = round_up(slab_tokens < SLAB_UNIT ? SLAB_UNIT : slab_tokens, SLAB_UNIT);
    const int64_t cap_eff = n_pad < cap ? n_pad : cap;
    p.slabs = plan_slabs(p.n, 1, 1, hdim, vocab, want_dw, slab_tokens, 2 * ((n_pad + cap_eff - 1) / cap_eff) + 1);
    Carver cv;
    p.off_slabs = cv.take(p.slabs.total);
    p.off_labels_eff = cv.take((size_t)p.n * sizeof(int64_t));
    p.off_mask = cv.take((size_t)p.n);
    p.off_cnt = cv.take((size_t)n_seqs * sizeof(int32_t));
    p.off_off = cv.take((size_t)n_seqs * sizeof(int32_t));
    p.off_seq_unsafe = cv.take((size_t)n_seqs);
    p.off_counts = cv.take((size_t)n_seqs * sizeof(float));
    p.off_dseq = cv.take((size_t)n_seqs * sizeof(float));
    p.off_gl = cv.take((size_t)p.bs * sizeof(float));
    p.total = cv.off;
    return p;
}
}  // namespace

extern "C" size_t oi_lmhead_dpo_workspace_bytes(int64_t n_seqs, int64_t total, int packed, int64_t hidden_dim,
                                                int64_t vocab, int want_d_weight, int64_t slab_tokens) {
    if (n_seqs <= 0 || total <= 0 || hidden_dim <= 0 || vocab <= 0 || slab_tokens <= 0) return 0;
    return plan_dpo(n_seqs, total, packed != 0, hidden_dim, vocab, want_d_weight != 0, slab_tokens).total;
}

extern "C" int oi_lmhead_dpo_fwd_bwd(const void* hidden, const void* weight, const int64_t* labels,
                                     const int32_t* cu_seq_lens, int64_t n_seqs, int64_t total, int64_t hidden_dim,
                                     int64_t vocab, float inv_temperature, const float* ref_chosen,
                                     const float* ref_rejected, float beta, float label_smoothing, float margin,
                                     int average_log_prob, float grad_scale, float* per_token_logps, float* seq_logps,
                                     float* losses, float* chosen_rewards, float* rejected_rewards, void* d_hidden,
                                     void* d_weight, int64_t slab_tokens, void* workspace, size_t workspace_bytes,
                                     void* stream) {
    OI_RETURN_IF(n_seqs < 2 || n_seqs % 2 != 0 || total < 1 || slab_tokens <= 0, OI_EINVAL);
    OI_RETURN_IF(n_seqs > MAX_LD || total > MAX_LD, OI_EINVAL);
    const bool packed = cu_seq_lens != nullptr;
    const int64_t n_tokens = packed ? total : n_seqs * total;
    int rc = check_lmhead(hidden, weight, labels, n_tokens, hidden_dim, vocab, inv_temperature);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF((ref_chosen == nullptr) != (ref_rejected == nullptr), OI_EINVAL);
    OI_RETURN_IF(!per_token_logps || !seq_logps || !losses || !d_hidden || !workspace, OI_ENULL);
    OI_RETURN_IF(!oi_aligned(workspace, 256) || !oi_aligned(d_hidden, 4) || !oi_aligned(d_weight, 4), OI_EALIGN);
    const DpoPlan p = plan_dpo(n_seqs, total, packed, hidden_dim, vocab, d_weight != nullptr, slab_tokens);
    OI_RETURN_IF(workspace_bytes < p.total, OI_EWORKSPACE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    char* ws = static_cast<char*>(workspace);
    char* ws_slabs = ws + p.off_slabs;
    int64_t* labels_eff = reinterpret_cast<int64_t*>(ws + p.off_labels_eff);
    uint8_t* mask = reinterpret_cast<uint8_t*>(ws + p.off_mask);
    int32_t* cnt = reinterpret_cast<int32_t*>(ws + p.off_cnt);
    int32_t* off = reinterpret_cast<int32_t*>(ws + p.off_off);
    uint8_t* seq_unsafe = reinterpret_cast<uint8_t*>(ws + p.off_seq_unsafe);
    float* counts = reinterpret_cast<float*>(ws + p.off_counts);
    float* d_seq = reinterpret_cast<float*>(ws + p.off_dseq);
    float* grad_losses = reinterpret_cast<float*>(ws + p.off_gl);
    float* grad = reinterpret_cast<float*>(ws_slabs + p.slabs.off_grad);
    uint8_t* unsafe = reinterpret_cast<uint8_t*>(ws_slabs + p.slabs.off_unsafe);
    const int64_t bs = p.bs;

    hipLaunchKernelGGL(dpo_rows_kernel, dim3((unsigned)n_seqs), dim3(256), 0, s, labels, cu_seq_lens, n_seqs, total,
                       labels_eff, mask, cnt);
    hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((bs + 63) / 64)), dim3(64), 0, s, grad_losses, bs, grad_scale);
    const SlabStep st = {hidden, weight, labels_eff, mask, n_tokens, hidden_dim, vocab, inv_temperature, per_token_logps,
                         nullptr, d_hidden, d_weight};
    // per-sequence sums of the logprobs computed so far, the loss derivative of every pair, and from it
    // every token's d loss / d logprob (right for the pairs whose tokens are all there)
    auto upstream = [&](bool) {
        int r = oi_seq_logp_fwd(per_token_logps, labels, cu_seq_lens, n_seqs, total, average_log_prob, seq_logps, counts,
                                stream);
        if (r != OI_OK) return r;
        r = oi_dpo_sigmoid_bwd(seq_logps, seq_logps + bs, ref_chosen, ref_rejected, nullptr, grad_losses, bs, beta,
                               label_smoothing, margin, d_seq, d_seq + bs, stream);
        if (r != OI_OK) return r;
        return oi_seq_logp_bwd(d_seq, labels, cu_seq_lens, counts, n_seqs, total, average_log_prob, grad, stream);
    };
    rc = run_slab_passes(
        p.slabs, ws_slabs, st, s,
        [&](int32_t* order, int32_t* count, SlabMeta* meta) {
            hipLaunchKernelGGL(dpo_plan_kernel, dim3(1), dim3(1), 0, s, cnt, (int)n_seqs, (int)p.slabs.cap,
                               (int)p.slabs.n_passes, off, seq_unsafe, count, meta);
            hipLaunchKernelGGL(dpo_order_kernel, dim3((unsigned)n_seqs), dim3(256), 0, s, mask, cu_seq_lens, n_seqs, total,
                               off, seq_unsafe, order, unsafe);
        },
        upstream);
    if (rc != OI_OK) return rc;
    // the sums are those of the last upstream pass (every logprob was there); losses and rewards from them
    return oi_dpo_sigmoid_fwd(seq_logps, seq_logps + bs, ref_chosen, ref_rejected, nullptr, bs, beta, label_smoothing,
                              margin, losses, chosen_rewards, rejected_rewards, stream);
}

extern "C" int oi_lmhead_probe_arm(int kernel) {
    OI_RETURN_IF(kernel < 0 || kernel > 2 || g_probe.kernel >= 0, OI_EINVAL);
    for (int i = 0; i < 2 * Probe::MAX_LAUNCHES; ++i) {
        const hipError_t e = hipEventCreate(&g_probe.ev[i]);
        if (e != hipSuccess) {
            for (int j = 0; j < i; ++j) (void)hipEventDestroy(g_probe.ev[j]);
            return (int)e;
        }
    }
    g_probe.used = 0;
    g_probe.kernel = kernel;
    return OI_OK;
}

extern "C" int oi_lmhead_probe_read(float* ms, int capacity, int* n_launches) {
    OI_RETURN_IF(g_probe.kernel < 0 || capacity < 0, OI_EINVAL);
    OI_RETURN_IF(!n_launches || (capacity > 0 && !ms), OI_ENULL);
    const int n = g_probe.used < capacity ? g_probe.used : capacity;
    int rc = OI_OK;
    for (int i = 0; i < n && rc == OI_OK; ++i) {
        hipError_t e = hipEventSynchronize(g_probe.ev[2 * i + 1]);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms[i], g_probe.ev[2 * i], g_probe.ev[2 * i + 1]);
        if (e != hipSuccess) rc = (int)e;
    }
    *n_launches = g_probe.used;
    for (int i = 0; i < 2 * Probe::MAX_LAUNCHES; ++i) (void)hipEventDestroy(g_probe.ev[i]);
    g_probe.kernel = -1;
    g_probe.used = 0;
    return rc;
}

extern "C" int oi_gemm_bf16_tn(const void* A, int64_t lda, int64_t M, const void* B, int64_t ldb, int64_t N, int64_t K,
                               float* out_f32, void* out_bf16, int64_t ldo, int accumulate, void* stream) {
    OI_RETURN_IF(M <= 0 || N <= 0 || K <= 0 || K % 64 != 0 || ldo < N, OI_EINVAL);
    OI_RETURN_IF(lda < 0 || ldb < 0 || lda % 8 != 0 || ldb % 8 != 0, OI_EINVAL);
    OI_RETURN_IF((lda != 0 && lda < K) || (ldb != 0 && ldb < K), OI_EINVAL);
    OI_RETURN_IF(lda > MAX_LD || ldb > MAX_LD, OI_EINVAL);
    OI_RETURN_IF(!A || !B || (!out_f32 && !out_bf16) || (out_f32 && out_bf16), OI_ENULL);
    OI_RETURN_IF(accumulate && !out_f32, OI_EINVAL);
    OI_RETURN_IF(!oi_aligned(A, 16) || !oi_aligned(B, 16), OI_EALIGN);
    // bf16 rows of even pitch are written as pairs (4-byte words), fp32 results as single words
    OI_RETURN_IF(!oi_aligned(out_f32, 4) || !oi_aligned(out_bf16, (ldo & 1) ? 2 : 4), OI_EALIGN);
    const int mode = out_f32 ? (accumulate ? 1 : 0) : 2;
    const Operand a = {static_cast<const uint16_t*>(A), lda, 0, M, K};
    const Operand b = {static_cast<const uint16_t*>(B), ldb, 0, N, K};
    hipLaunchKernelGGL((gemm_store_kernel<false, false>), dim3(grid_for_tiles((M + BM - 1) / BM, (N + BN - 1) / BN)),
                       dim3(NTHREADS), 0, static_cast<hipStream_t>(stream), a, M, b, N, K, mode, out_f32,
                       static_cast<uint16_t*>(out_bf16), ldo, M, DynRows{nullptr, 0, nullptr, nullptr, nullptr, nullptr}, static_cast<uint32_t*>(nullptr));
    return oi_launch_status();
}

extern "C" int oi_gemm_bf16_layouts(const void* A, int64_t lda, int a_k_major, const void* B, int64_t ldb,
                                    int b_k_major, int64_t M, int64_t N, int64_t K, float* out_f32, void* out_bf16,
                                    int64_t ldo, int accumulate, void* stream) {
    OI_RETURN_IF(M <= 0 || N <= 0 || K <= 0 || K % 64 != 0 || ldo < N, OI_EINVAL);
    OI_RETURN_IF(lda <= 0 || ldb <= 0 || lda % 8 != 0 || ldb % 8 != 0 || lda > MAX_LD || ldb > MAX_LD, OI_EINVAL);
    // a k-major operand is read in 16-byte column chunks: whole chunks only
    OI_RETURN_IF(lda < (a_k_major ? M : K) || ldb < (b_k_major ? N : K), OI_EINVAL);
    OI_RETURN_IF((a_k_major && M % 8 != 0) || (b_k_major && N % 8 != 0), OI_EINVAL);
    OI_RETURN_IF(!A || !B || (!out_f32 && !out_bf16) || (out_f32 && out_bf16), OI_ENULL);
    OI_RETURN_IF(accumulate && !out_f32, OI_EINVAL);
    OI_RETURN_IF(!oi_aligned(A, 16) || !oi_aligned(B, 16), OI_EALIGN);
    // bf16 rows of even pitch are written as pairs (4-byte words), fp32 results as single words
    OI_RETURN_IF(!oi_aligned(out_f32, 4) || !oi_aligned(out_bf16, (ldo & 1) ? 2 : 4), OI_EALIGN);
    const int mode = out_f32 ? (accumulate ? 1 : 0) : 2;
    const Operand a = {static_cast<const uint16_t*>(A), lda, 0, M, K};
    const Operand b = {static_cast<const uint16_t*>(B), ldb, 0, N, K};
    const dim3 grid(grid_for_tiles((M + BM - 1) / BM, (N + BN - 1) / BN));
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint16_t* o16 = static_cast<uint16_t*>(out_bf16);
    uint32_t* no_queue = nullptr;
    const DynRows fixed = {nullptr, 0, nullptr, nullptr, nullptr, nullptr};
    if (a_k_major && b_k_major)
        hipLaunchKernelGGL((gemm_store_kernel<true, true>), grid, dim3(NTHREADS), 0, s, a, M, b, N, K, mode, out_f32, o16,
                           ldo, M, fixed, no_queue);
    else if (a_k_major)
        hipLaunchKernelGGL((gemm_store_kernel<true, false>), grid, dim3(NTHREADS), 0, s, a, M, b, N, K, mode, out_f32,
                           o16, ldo, M, fixed, no_queue);
    else if (b_k_major)
        hipLaunchKernelGGL((gemm_store_kernel<false, true>), grid, dim3(NTHREADS), 0, s, a, M, b, N, K, mode, out_f32,
                           o16, ldo, M, fixed, no_queue);
    else
        hipLaunchKernelGGL((gemm_store_kernel<false, false>), grid, dim3(NTHREADS), 0, s, a, M, b, N, K, mode, out_f32,
                           o16, ldo, M, fixed, no_queue);
    return oi_launch_status();
}

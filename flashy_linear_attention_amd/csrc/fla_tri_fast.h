// Fast path of Out = mask(X Y^T) Z for 16-byte aligned operands.
//
// Same mathematics and the same MFMA operand chaining as fla_tri_kernel.h (S^T
// accumulators feed the second product straight from registers, Z is read with
// ds_read_b64_tr_b16).  What differs is how data moves and how the loop is
// pipelined:
//
//   * Y/Z tiles (BN = 64 rows) go HBM -> LDS with buffer_load_dwordx4 ... lds
//     (no staging registers, no ds_write), into a ring of three to five LDS
//     slots.  One wave instruction fills 1 KiB of LDS in lane order, so the bank
//     spreading that padding would give is done by an XOR swizzle of the
//     16-byte chunk index instead: a lane fetches the global chunk that belongs
//     at its LDS slot.  Rows beyond N and chunks beyond the real width are
//     pointed outside the buffer resource and arrive as zeros.
//   * The walk over tiles that lie entirely inside the mask is software
//     pipelined per 32-row sub-tile s, with no masking code at all:
//         phase 1:  S_s = Y_s X^T       | fetch Z fragments of s-1 from LDS
//         phase 2:  Out += P_{s-1} Z_{s-1} | fetch Y fragments of s+1, round S_s to P_s
//     so every LDS read is issued about half an iteration (~500 cycles) before
//     its MFMA and the two MFMA chains of a phase are independent.
//     One barrier per tile, placed between the phases of the tile's second
//     sub-tile: it publishes the next tile and retires the previous one.
//     With one wave per SIMD a wave issues one instruction every four clocks and
//     an MFMA holds the pipe for 32, so at most seven other instructions fit
//     between two MFMAs: the loads of the tile that goes into the retired slot
//     are issued one per MFMA group of the following phase, with their scalar
//     offsets computed beforehand, unconditionally (a tile past the end of the
//     sequence is fetched from out of range) so that no branch or variable wait
//     count sits in the loop.
//   * The BM x BM block on the diagonal is handled afterwards, with all of its
//     tiles resident, by a barrier-free S -> mask -> P -> PV sequence per sub-tile
//     that skips the (block, sub-tile) pairs the mask removes entirely.
//   * A workgroup does two row tiles (r and n_tiles-1-r).  The second one's first
//     tile and X fragments are requested before the first one's epilogue, into
//     ring slots behind the epilogue's staging area.
//   * Variants of the same body: the plain kernel (one product), the batched
//     kernel (grid y selects one of up to three products: the backward's dQ, dV,
//     dK in one launch) and the chunked kernel (CHUNKED: diagonal block plus
//     the running state of the chunk-wise evaluation, no tile ring).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "fla_feature.h"
#include "fla_tri_kernel.h"

namespace fla {

typedef __attribute__((address_space(3))) void *lds_void_ptr;
typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
typedef short s16x8 __attribute__((ext_vector_type(8)));

// One wave-wide HBM -> LDS copy of 64 x 16 bytes: lane l's 16 bytes land at lds_addr + 16 l.
// Issued through inline assembly so that the compiler's wait-count insertion does not
// serialise later LDS reads of *other* ring slots against it; completion is awaited
// explicitly (wait_dma) before the barrier that publishes the slot.
// The LDS address is lds_base + LDS_IMM with LDS_IMM a compile-time constant, added while M0 is
// written: the loads of one tile then need a single scalar base between them.
template <int LDS_IMM>
__device__ __forceinline__ void dma_16B_per_lane(u32x4 rsrc, uint32_t lds_base, uint32_t voffset, uint32_t soffset) {
    asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset), "n"(LDS_IMM)
                 : "memory", "m0", "scc");
}
// s_waitcnt vmcnt(N) only (expcnt and lgkmcnt fields left at their maxima): returns once at
// most N of this wave's buffer loads, the most recently issued ones, are still in flight.
// f(integral_constant<int, I>) for I = BEGIN .. END-1, unrolled at compile time
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}
template <int N>
__device__ __forceinline__ void wait_vm() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

__device__ __forceinline__ u32x4 make_rsrc(const void *base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    u32x4 r = {(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, bytes, 0x00020000u};
    return r;
}

// Two fp32 values rounded (nearest even) and packed into one 16-bit pair, pinned to this
// point of the instruction stream.  As a plain conversion the compiler sinks all sixteen of a
// sub-tile to just before the first MFMA that reads the result, where they leave the matrix
// pipe idle.  The empty volatile asm statement demands the result right here, and the
// scheduling barriers around the caller keep it from moving up; the conversion itself stays
// a compiler-generated instruction, so that the hazard recogniser still sees it next to the
// MFMAs that produce and consume these registers (hand-written conversion instructions in
// inline assembly gave wrong results: the required wait states were missing).
template <typename T>
__device__ __forceinline__ uint32_t round_pack_pinned(float lo, float hi) {
    typedef T pair_t __attribute__((ext_vector_type(2)));
    pair_t pr;
    pr[0] = static_cast<T>(lo);
    pr[1] = static_cast<T>(hi);
    uint32_t r = __builtin_bit_cast(uint32_t, pr);
    asm volatile("" : "+v"(r));
    return r;
}

constexpr uint32_t kOobOffset = 0x40000000u;  // added to a buffer offset to force an out-of-range (zero) access
constexpr int64_t kMaxFastExtent = 0x3fffffff;  // per-(b,h) byte extent the 32-bit buffer offsets can address

constexpr int kSwizzlePeriodY = 16;  // rows after which swizzle_y (below) repeats

// CHUNKED = false: the quadratic walk over all tiles under the mask; true: chunk-wise evaluation
// (diagonal block plus running state), compiled as a kernel of its own.
template <int DC, int DO, bool CHUNKED = false>
struct FastConfig {
    static constexpr int MW = TriConfig<DC, DO>::MW;
    static constexpr int NW = 4;
    static constexpr int BM = MW * NW;
    static constexpr int BN = 64;
    static constexpr int RY = DC * 2, RZ = DO * 2;  // LDS row bytes (no padding)
    static constexpr int CY = DC / 8, CZ = DO / 8;  // 16-byte chunks per row
    static constexpr int Y_BYTES = BN * RY, Z_BYTES = BN * RZ;
    static constexpr int STAGE_BYTES = Y_BYTES + Z_BYTES;
    // LDS ring depth.  Quadratic walk: the tile being consumed, the one before it (its second
    // half is still being read for a while) and NBUF-2 tiles landed or in flight: as many as
    // fit, up to five (with five, the whole diagonal block is on its way when the walk over the
    // full tiles ends).  Chunked: exactly the tiles of the diagonal block, nothing cycles.
    static constexpr int kMaxSlots = (160 * 1024) / STAGE_BYTES;
    static constexpr int NBUF = CHUNKED ? BM / BN : (kMaxSlots >= 5 ? 5 : kMaxSlots);
    static constexpr int SMEM_BYTES = NBUF * STAGE_BYTES;
    static constexpr bool kSupported = kMaxSlots >= 3 && BM / BN <= kMaxSlots;
    // chunked evaluation: the running state S^T, [DO rows][DC] 16-bit, sits behind the tiles in
    // whole 64-row units of the Y tile layout when the 160 KiB allow it
    static constexpr int STATE_BYTES = ((DO + 63) / 64) * Y_BYTES;
    static constexpr bool kStateInLds = CHUNKED && SMEM_BYTES + STATE_BYTES <= 160 * 1024;
    // the transposed state ([DC rows][DO], Z tile layout) is read only by square instantiations
    static constexpr bool kStateTransposable = kStateInLds && DC == DO;
    // Narrow shapes need half the LDS and about half the registers: holding the kernel to 256
    // registers lets two workgroups share a CU, which hides each other's prologue and epilogue.
    static constexpr int kMinWavesPerSimd = (DC <= 64 && DO <= 64) ? 2 : 1;
    // wave-level 1 KiB DMA instructions per tile and wave
    static constexpr int NIY = Y_BYTES / 4096, NIZ = Z_BYTES / 4096;
    static constexpr int NT = NIY + NIZ;  // buffer loads per wave and tile
    // distinct per-lane source offsets among the Y loads of a tile (see swizzle_y)
    static constexpr int NYD = (4 * (1024 / RY)) % kSwizzlePeriodY == 0 ? 1 : 2;
    static_assert((NYD * 4 * (1024 / RY)) % kSwizzlePeriodY == 0 && (NIY % NYD) == 0, "Y swizzle period");
    // output staging in LDS: BM rows of DO 16-bit values, 16 bytes of padding per row
    static constexpr int RO = DO * 2 + 16;
    static_assert(BM * RO <= SMEM_BYTES, "output staging must fit in the ring");
    static_assert(Y_BYTES % 4096 == 0 && Z_BYTES % 4096 == 0, "tile must split into 1 KiB blocks over 4 waves");
};

// XOR applied to the chunk index of LDS row `row` (row counted inside the tile).
// Y: a 16-byte-per-lane read is served 16 lanes at a time out of 64 banks of 4 bytes, and the 16
// lanes read one chunk index of 16 consecutive rows: the 16 rows must land in the 16 different
// 16-byte slots of a 256-byte window (measured: 4-5 clocks per instruction then, 8 with only 8
// slots covered).  Rows of 256 bytes and more all start at bank 0, so the row's low 4 bits go
// into the chunk index; with 128- / 64-byte rows the low 1 / 2 row bits already pick a different
// part of the window and the next 3 / 2 bits are folded in.
template <int CY>
__device__ __forceinline__ int swizzle_y(int row) {
    if constexpr (CY == 4) return (row >> 2) & 3;
    else if constexpr (CY == 8) return (row >> 1) & 7;
    else return row & 15;
}
template <int CZ>
__device__ __forceinline__ int swizzle_z(int row) {
    if constexpr (CZ == 4) return ((row >> 1) & 1) << 1;
    else return (row & 3) << 1;  // the 4 rows of one transposing read land in 4 different 32-byte slots
}

// The work of one workgroup; `wg_index` is its index within one product's grid.
// FLAGS of the quadratic walk: kNormFlag divides each output row by the sum of its masked scores
// (the normaliser of linear attention); kPolyFlag maps every score through a quadratic polynomial
// (second-order Taylor feature map without the features).
// kDualFlag: two scores from one pass over the contraction -- columns [0, D_c/2) of X and Y give
// u1, columns [D_c/2, D_c/2 + 32) give u2, and the score is u1 (poly[0] + poly[1] u2 + poly[2] u2^2):
// the gradient of the polynomial score map with respect to its argument, e.g.
// lower((dO V^T) . f'(Xq Xk^T)) Xk with X = [dO | xq] and Y = [V | xk] packed side by side.
// kTailFlag (with kDualFlag): the second operand sits in the last 32 columns of the padded
// contraction instead, [D_c - 32, D_c), which leaves the first one D_c - 32 columns -- room for an
// extra column that adds a per-row bias to u1 ([.. | b_i] . [.. | 1]).
constexpr int kNormFlag = 1, kPolyFlag = 2, kDualFlag = 4, kTailFlag = 8;
constexpr int kPolyMaxContraction = 64;  // polynomial variants are built for D_c <= 64 only

template <typename T, int DC, int DO, bool CHUNKED, int FLAGS = 0>
__device__ __forceinline__ void tri_fast_body(const TriParams &p, const int wg_index) {
    constexpr bool NORM = (FLAGS & kNormFlag) != 0, POLY = (FLAGS & kPolyFlag) != 0, DUAL = (FLAGS & kDualFlag) != 0;
    static_assert(!(DUAL && (POLY || NORM)), "the dual-score walk has its own score map and no normaliser");
    static_assert(!DUAL || DC >= 64, "the dual-score walk needs room for two contractions");
    static_assert(!(CHUNKED && FLAGS != 0), "score maps and the in-kernel normaliser belong to the quadratic walk");
    // The body is compiled in the device pass only: hipcc's host pass silently
    // drops the launch stub of a kernel template whose body calls the LDS-DMA
    // builtin from inside a lambda, and the host needs nothing but the stub.
#if defined(__HIP_DEVICE_COMPILE__)
    using Cfg = FastConfig<DC, DO, CHUNKED>;
    using M = Mma<T>;
    using V8 = typename M::V8;
    constexpr int MW = Cfg::MW, BM = Cfg::BM, BN = Cfg::BN;
    constexpr int NIB = MW / 32, NBLK = BM / 32;
    constexpr int KC = DC / 16, DB = DO / 32, NZF = 2 * DB;
    constexpr int RY = Cfg::RY, RZ = Cfg::RZ, CY = Cfg::CY, CZ = Cfg::CZ;
    constexpr int NIY = Cfg::NIY, NIZ = Cfg::NIZ;
    constexpr int STAGE = Cfg::STAGE_BYTES, Y_BYTES = Cfg::Y_BYTES;
    // chunks of the contraction that feed the first score / that are used at all (DUAL: the
    // second score takes two chunks, 32 columns, right after the first half)
    constexpr bool TAIL = (FLAGS & kTailFlag) != 0;
    static_assert(!TAIL || DUAL, "the tail layout is a layout of the dual-score walk");
    constexpr int KC1 = !DUAL ? KC : TAIL ? KC - 2 : KC / 2, KCU = (DUAL && !TAIL) ? KC / 2 + 2 : KC;
    constexpr int YQ = KC < 8 ? KC : 8;  // Y read addresses that differ by more than an immediate
    constexpr int ZQ = DB < 2 ? DB : 2;  // same for Z

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, g = lane >> 5, lam = lane & 15;

    const int wg = wg_index, xcd = wg & 7, slot = wg >> 3;
    // Each workgroup takes two row tiles of one head, r and n_tiles-1-r: under a triangular
    // mask their work adds up to the same amount for every r, so all workgroups are equal.
    // (Chunked evaluation: one row tile per workgroup, all of equal work already.)
    constexpr bool chunked = CHUNKED;
    const bool single = chunked || p.single != 0;
    const int n_pairs = single ? p.n_tiles : (p.n_tiles + 1) >> 1;
    // Pairs: the workgroups of one head are neighbours (they stream the same Y / Z rows at the
    // same time).  Single tiles differ in work, so they are ordered heaviest first across all
    // heads: whatever CU frees up next takes the heaviest tile left.
    const int n_hl = (p.BH + 7) >> 3;
    const int hl = (single && !chunked) ? slot % n_hl : slot / n_pairs;
    const int rank = (single && !chunked) ? slot / n_hl : slot - hl * n_pairs;
    const int bh = hl * 8 + xcd;
    if (bh >= p.BH) return;
    const bool upper = p.upper != 0;
    const int b = bh / p.H, h = bh - b * p.H;
    const T *X = static_cast<const T *>(p.x) + b * p.xs_b + h * p.xs_h;
    const T *Y = static_cast<const T *>(p.y) + b * p.ys_b + h * p.ys_h;
    const T *Z = static_cast<const T *>(p.z) + b * p.zs_b + h * p.zs_h;
    T *O = static_cast<T *>(p.out) + b * p.os_b + h * p.os_h;
    const int N = p.N;

    // raw buffer resources covering exactly the valid rows of this (b, h)
    const int xs2 = (int)p.xs_n * 2, ys2 = (int)p.ys_n * 2, zs2 = (int)p.zs_n * 2;
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(X), 0, (N - 1) * xs2 + p.dc * 2, 0x00020000);
    const u32x4 ry = make_rsrc(Y, (uint32_t)((N - 1) * ys2 + p.dc * 2));
    const u32x4 rz = make_rsrc(Z, (uint32_t)((N - 1) * zs2 + p.dout * 2));

    int blk[NIB];
    blk[0] = wave;
    if constexpr (NIB == 2) blk[1] = NBLK - 1 - wave;

    // ---- the row tiles of this workgroup, in the order they are done: unpaired tiles go heaviest
    // first (last row tile under a lower mask, first under an upper one); with an odd tile
    // count the middle tile has no partner; chunked: a single tile per workgroup
    auto stream_tile = [&](int pass) {
        return chunked ? rank : single ? (upper ? rank : p.n_tiles - 1 - rank) : (pass == 0 ? p.n_tiles - 1 - rank : rank);
    };
    const int n_pass = (single || rank == p.n_tiles - 1 - rank) ? 1 : 2;
    // geometry of the tile being set up; the tile sequence is the tiles fully inside the mask
    // first, then the diagonal block
    int tile = 0, i0 = 0, diag_rows = 0, n_diag = 0, n_full = 0, full_row0 = 0, n_seq = 0;
    auto set_tile = [&](int t) {
        tile = t;
        i0 = t * BM;
        diag_rows = (N - i0 < BM) ? (N - i0) : BM;
        n_diag = (diag_rows + BN - 1) / BN;
        if (upper) {
            const int rest = N - (i0 + BM);
            n_full = rest > 0 ? (rest + BN - 1) / BN : 0;
            full_row0 = i0 + BM;
        } else {
            n_full = i0 / BN;
            full_row0 = 0;
        }
        if (chunked) n_full = 0;  // everything off the diagonal block arrives through the state
        n_seq = n_full + n_diag;
    };

    // ---- HBM -> LDS: per-lane source offsets (constant over tiles).  Load u of a wave covers
    // rows u * YSTEP + wave * (1024 / RY) + lane / CY of the tile.  Where YSTEP is a multiple of
    // the swizzle period the lane's chunk is the same for every u and the row advance goes into
    // the scalar offset: one address register per operand, no vector work per load (512-byte Y
    // rows: the period is two steps, so two registers, for even and odd u).
    constexpr int YSTEP = 4 * (1024 / RY), ZSTEP = 4 * (1024 / RZ);
    constexpr int NYD = Cfg::NYD;
    static_assert(NIZ == 1 || ZSTEP % 4 == 0, "Z swizzle must not depend on the load index");
    uint32_t ydma[NYD], zdma;
#pragma unroll
    for (int v = 0; v < NYD; ++v) {
        const int row = v * YSTEP + wave * (1024 / RY) + lane / CY;
        const int c = (lane % CY) ^ swizzle_y<CY>(row);
        ydma[v] = (uint32_t)(row * ys2 + c * 16) + (c * 8 < p.dc ? 0u : kOobOffset);
    }
    {
        const int row = wave * (1024 / RZ) + lane / CZ;
        const int c = (lane % CZ) ^ swizzle_z<CZ>(row);
        zdma = (uint32_t)(row * zs2 + c * 16) + (c * 8 < p.dout ? 0u : kOobOffset);
    }
    const uint32_t lds_wave = lds0 + wave * 1024;
    // tile q of the sequence -> ring slot q % NBUF, tracked incrementally by the caller
    auto tile_row0 = [&](int q) { return q < n_full ? full_row0 + q * BN : i0 + (q - n_full) * BN; };
    // load I of the NT wave-level loads of a tile, into the slot at yb
    auto issue_part_at = [&](auto ii, uint32_t soffset, uint32_t yb) {
        constexpr int I = decltype(ii)::value;
        if constexpr (I < NIY)
            dma_16B_per_lane<I * 4096>(ry, yb, ydma[I % NYD], soffset);
        else
            dma_16B_per_lane<Y_BYTES + (I - NIY) * 4096>(rz, yb, zdma, soffset);
    };
    // Scalar offsets of the NT loads of tile q.  A tile past the end of the sequence is loaded
    // all the same, from out of range: zeros arrive in a slot nobody reads (callers only name
    // slots that are free), and the count of loads in flight is the same at every step, which
    // keeps branches out of the instruction stream and makes wait_tile a constant.
    auto tile_offsets = [&](int q, uint32_t (&so)[Cfg::NT]) {
        const bool exists = q < n_seq;
        const int row0 = tile_row0(q);
        const uint32_t ybase = exists ? (uint32_t)(row0 * ys2) : kOobOffset;
        const uint32_t zbase = exists ? (uint32_t)(row0 * zs2) : kOobOffset;
        static_for<0, Cfg::NT>([&](auto ii) {
            constexpr int I = decltype(ii)::value;
            so[I] = I < NIY ? ybase + (uint32_t)((I - I % NYD) * YSTEP * ys2) : zbase + (uint32_t)((I - NIY) * ZSTEP * zs2);
        });
    };
    auto issue_tile = [&](int q, int slot_off) {
        uint32_t so[Cfg::NT];
        tile_offsets(q, so);
        const uint32_t yb = lds_wave + slot_off;
        static_for<0, Cfg::NT>([&](auto ii) { issue_part_at(ii, so[decltype(ii)::value], yb); });
    };
    auto next_slot = [](int off) { return off + STAGE == Cfg::NBUF * STAGE ? 0 : off + STAGE; };
    // Wait until a tile has landed, given that exactly the NBUF - 3 tiles after it have been
    // issued since: their loads may stay in flight.
    auto wait_tile = [&]() {
        constexpr int AHEAD = Cfg::NBUF > 3 ? Cfg::NBUF - 3 : 0;
        static_assert(AHEAD * Cfg::NT < 64, "vmcnt is a 6-bit field");
        wait_vm<AHEAD * Cfg::NT>();
    };

    constexpr int RING = Cfg::NBUF * STAGE;
    auto wrap_slot = [](int off) { return off >= RING ? off - RING : off; };

    // ---- resident X fragments
    V8 xf[NIB][KC];
    auto load_x = [&]() {
#pragma unroll
        for (int ib = 0; ib < NIB; ++ib) {
            const int row = i0 + blk[ib] * 32 + l32;
#pragma unroll
            for (int kc = 0; kc < KCU; ++kc) {
                const int col = kc * 16 + 8 * g;
                const uint32_t off = (uint32_t)(row * xs2 + col * 2) + (col < p.dc ? 0u : kOobOffset);
                xf[ib][kc] = __builtin_bit_cast(V8, __builtin_amdgcn_raw_buffer_load_b128(rx, off, 0, 0));
            }
        }
    };
    // First requests of a row tile: tile 0 of its sequence, the X fragments, then tiles up to
    // kPre - 1, into ring slots starting at byte offset ring0.  For the second row tile of a
    // workgroup this runs before the first one's epilogue (kOverlap): the epilogue stages the
    // output in the first kStageSlots slots, the requests go to the slots behind them, and the
    // latency of the first loads is hidden behind the epilogue.
    constexpr int kStageSlots = (BM * Cfg::RO + STAGE - 1) / STAGE;
    constexpr int kFreeSlots = Cfg::NBUF - kStageSlots;
    constexpr bool kOverlap = !CHUNKED && kFreeSlots >= 1 && Cfg::NBUF >= 3;
    constexpr int kPre = 1;  // (two tiles up front measured no better than one)
    static_assert(kPre >= 1, "tile 0 is always requested up front");
    int ring0 = 0;
    auto start_tile = [&]() {
        issue_tile(0, ring0);
        load_x();
        static_for<1, kPre>([&](auto qq) { issue_tile(decltype(qq)::value, wrap_slot(ring0 + decltype(qq)::value * STAGE)); });
    };
    set_tile(stream_tile(0));
    start_tile();

    for (int pass = 0;; ++pass) {

    f32x16 acc[NIB][DB];
#pragma unroll
    for (int ib = 0; ib < NIB; ++ib)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[ib][db][v] = 0.f;
    // NORM: running sum of this lane's masked scores per row block (row l32, the 16 key rows of
    // every sub-tile that fall to this half-wave); the two halves are added in the epilogue
    float rsum[NIB];
#pragma unroll
    for (int ib = 0; ib < NIB; ++ib) rsum[ib] = 0.f;
    const float pc0 = p.poly[0], pc1 = p.poly[1], pc2 = p.poly[2];
    auto map_scores = [&](f32x16 &sc) {
#pragma unroll
        for (int v = 0; v < 16; ++v) sc[v] = __builtin_fmaf(__builtin_fmaf(pc2, sc[v], pc1), sc[v], pc0);
    };
    auto combine_scores = [&](f32x16 &sc, const f32x16 &sc2) {
#pragma unroll
        for (int v = 0; v < 16; ++v) sc[v] *= __builtin_fmaf(__builtin_fmaf(pc2, sc2[v], pc1), sc2[v], pc0);
    };
    auto add_scores = [&](const f32x16 &sc, float &dst) {
        float t0 = (sc[0] + sc[1]) + (sc[2] + sc[3]), t1 = (sc[4] + sc[5]) + (sc[6] + sc[7]);
        float t2 = (sc[8] + sc[9]) + (sc[10] + sc[11]), t3 = (sc[12] + sc[13]) + (sc[14] + sc[15]);
        dst += (t0 + t1) + (t2 + t3);
    };

    // ---- LDS read offsets inside a stage.  Only the chunk bits the swizzle touches need a
    // register; the rest of (sub-tile, kc / t, db) is an immediate offset of the DS instruction.
    int ylane[YQ], zlane[ZQ];
    {
        const int sy = swizzle_y<CY>(l32);
#pragma unroll
        for (int j = 0; j < YQ; ++j) ylane[j] = l32 * RY + (((2 * j + g) ^ sy) << 4);
        // Transposing read: source lane `lam` of a 16-lane group supplies row lam/4 and the
        // 4-column chunk c = lam%4; destination lane 4c + x receives column x of that chunk.
        // Chunk c of group beta = (lane/16)%2 is taken from columns 16 (c&1) + 8 beta + 4 (c>>1)
        // of the 32-column block, which makes MFMA row m = 8a + 4g' + b of the fragment hold
        // column 16 g' + 4 a + b: the accumulator registers of one lane then cover 16
        // consecutive output columns (see the epilogue).
        const int zrow = 4 * g + (lam >> 2);
        const int sz = swizzle_z<CZ>(zrow);
        const int zc = lam & 3, beta = (lane >> 4) & 1;
#pragma unroll
        for (int j = 0; j < ZQ; ++j)
            zlane[j] = Y_BYTES + zrow * RZ + (((4 * j + 2 * (zc & 1) + beta) ^ sz) << 4) + 8 * (zc >> 1);
    }
    // `ya` / `za`: ylane / zlane plus the byte offset of a ring slot
    auto y_read = [&](const int (&ya)[YQ], int sub, int kc) -> V8 {
        const unsigned char *ptr = smem + ya[kc % YQ] + (sub * 32 * RY + (kc / YQ) * (YQ * 32));
        return __builtin_bit_cast(V8, *reinterpret_cast<const u32x4 *>(ptr));
    };
    // fragment f = (t, db): rows 16t + {4g..4g+3, 8+4g..} of sub-tile `sub`, columns of block db
    auto z_read = [&](const int (&za)[ZQ], int sub, int f) -> V8 {
        const int t = f / DB, db = f % DB;
        const unsigned char *zp = smem + za[db % ZQ] + ((sub * 32 + 16 * t) * RZ + (db / ZQ) * (ZQ * 64));
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(zp));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(zp + 8 * RZ));
        return __builtin_bit_cast(V8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    auto slot_addrs = [&](int slot_off, int (&ya)[YQ], int (&za)[ZQ]) {
#pragma unroll
        for (int j = 0; j < YQ; ++j) ya[j] = ylane[j] + slot_off;
#pragma unroll
        for (int j = 0; j < ZQ; ++j) za[j] = zlane[j] + slot_off;
    };
    auto round_p = [&](const f32x16 (&s)[NIB], V8 (&pf)[NIB][2]) {
#pragma unroll
        for (int ib = 0; ib < NIB; ++ib)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[ib][t][e] = static_cast<T>(s[ib][8 * t + e]);
    };

    // ring state: byte offsets of the slots of tile q-1, q, q+1 and of the next tile to issue
    int prev_off = wrap_slot(ring0 + (Cfg::NBUF - 1) * STAGE), cur_off = ring0, next_off = wrap_slot(ring0 + STAGE);
    // The last row block's X fragments are held in accumulation registers (MFMA reads its A / B
    // operands from there as well).  Left to itself the register allocator parks them there
    // anyway, the architectural file being full, but then copies each one to a second
    // accumulation register before every use: four moves per MFMA in the main loop.
    // (Only where a wave has the whole register file: with two waves per SIMD nothing is parked.
    // Placed after the first wait for loaded data: the statement needs the values.)
    auto pin_x = [&]() {
        if constexpr (Cfg::kMinWavesPerSimd == 1) {
#pragma unroll
            for (int kc = 0; kc < KCU; ++kc) asm volatile("" : "+a"(xf[NIB - 1][kc]));
        }
    };
    const bool has_state = chunked && (upper ? tile + 1 < p.n_tiles : tile > 0);
    const T *st = has_state ? static_cast<const T *>(p.state) + ((int64_t)bh * p.n_tiles + tile) * (DO * DC) : nullptr;
    if constexpr (chunked) {
        // The kernel is bound by its loads.  With two workgroups on a CU everything is requested at
        // once (the other workgroup computes meanwhile).  A workgroup that has the CU to itself
        // requests what the state product below needs first -- the X fragments and the running
        // state, with tile 0 -- and the other tiles once that has landed, so that the product runs
        // while they arrive: asked for together, all of it would arrive at the end.
        constexpr bool kLateTiles = Cfg::kMinWavesPerSimd == 1;
        if constexpr (!kLateTiles)
            static_for<kPre, BM / BN>([&](auto qq) { issue_tile(decltype(qq)::value, decltype(qq)::value * STAGE); });
        if constexpr (Cfg::kStateInLds) {
            if (has_state) {
                const u32x4 rs = make_rsrc(st, DO * DC * 2);
                if (Cfg::kStateTransposable && p.state_transposed) {
                    // [DC rows][DO] in the Z tile layout
                    const int row = wave * (1024 / RZ) + lane / CZ;
                    const uint32_t tdma = (uint32_t)(row * RZ + (((lane % CZ) ^ swizzle_z<CZ>(row)) << 4));
                    static_for<0, (DC + 63) / 64>([&](auto uu) {
                        constexpr int UNIT = decltype(uu)::value;
                        static_for<0, NIZ>([&](auto u) {
                            constexpr int U = decltype(u)::value;
                            dma_16B_per_lane<Cfg::SMEM_BYTES + UNIT * Cfg::Z_BYTES + U * 4096>(
                                rs, lds_wave, tdma, (uint32_t)((UNIT * 64 + U * ZSTEP) * RZ));
                        });
                    });
                } else {
                    // [DO rows][DC] in the Y tile layout
                    uint32_t sdma[NYD];
#pragma unroll
                    for (int v = 0; v < NYD; ++v) {
                        const int row = v * YSTEP + wave * (1024 / RY) + lane / CY;
                        sdma[v] = (uint32_t)(row * RY + (((lane % CY) ^ swizzle_y<CY>(row)) << 4));
                    }
                    static_for<0, Cfg::STATE_BYTES / Y_BYTES>([&](auto uu) {
                        constexpr int UNIT = decltype(uu)::value;
                        static_for<0, NIY>([&](auto u) {
                            constexpr int U = decltype(u)::value;
                            dma_16B_per_lane<Cfg::SMEM_BYTES + UNIT * Y_BYTES + U * 4096>(
                                rs, lds_wave, sdma[U % NYD], (uint32_t)((UNIT * 64 + (U - U % NYD) * YSTEP) * RY));
                        });
                    });
                }
            }
        }
        wait_vm<0>();
        __builtin_amdgcn_s_barrier();
        if (p.map_x) {
            // X = phi(x): the fragments are in registers (a lane holds eight consecutive columns of
            // one row per fragment); columns beyond the true width stay zero.  The mapped rows are
            // written out once, for the passes that need phi(x) later.
            T *XO = static_cast<T *>(p.xmap_out) + b * p.xo_b + h * p.xo_h;
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib) {
                const int row = i0 + blk[ib] * 32 + l32;
#pragma unroll
                for (int kc = 0; kc < KC; ++kc) {
                    const int col = kc * 16 + 8 * g;
                    if (col < p.dc) {
                        const u32x4 m = feature_map8<T>(p.map_x, __builtin_bit_cast(u32x4, xf[ib][kc]));
                        xf[ib][kc] = __builtin_bit_cast(V8, m);
                        if (row < N) *reinterpret_cast<u32x4 *>(XO + (int64_t)row * p.xo_n + col) = m;
                    }
                }
            }
        }
        pin_x();
        if constexpr (kLateTiles)
            static_for<kPre, BM / BN>([&](auto qq) { issue_tile(decltype(qq)::value, decltype(qq)::value * STAGE); });
    } else {
        // tiles up to NBUF-3 before the first wait, tile NBUF-2 right after it
        static_for<kPre, Cfg::NBUF - 2>(
            [&](auto qq) { issue_tile(decltype(qq)::value, wrap_slot(ring0 + decltype(qq)::value * STAGE)); });
        wait_tile();
        __builtin_amdgcn_s_barrier();  // tile 0 (and the X fragments) have landed
        pin_x();
        issue_tile(Cfg::NBUF - 2, wrap_slot(ring0 + (Cfg::NBUF - 2) * STAGE));
    }
    // from here on: tiles up to q + NBUF - 2 are issued while tile q is consumed, and tile
    // q + NBUF - 1 goes into the slot of tile q - 1 (prev_off) once that one is retired
    auto advance = [&]() {
        prev_off = cur_off;
        cur_off = next_off;
        next_off = next_slot(next_off);
    };
    int q = 0;

    // ================= tiles fully inside the mask: pipelined, no masking =================
    if (n_full > 0) {
        V8 yf[KC], zf[NZF], pfa[NIB][2], pfb[NIB][2];
        f32x16 s[NIB], s2[NIB];
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        {
            int ya0[YQ], za0[ZQ];
            slot_addrs(cur_off, ya0, za0);
#pragma unroll
            for (int kc = 0; kc < KCU; ++kc) yf[kc] = y_read(ya0, 0, kc);
        }

        // phase 1 of sub-tile s: S = Y_s X^T, interleaved with the Z fragment reads of the previous sub-tile
        auto phase1 = [&](auto with_z, const int (&za)[ZQ], int zsub) {
#pragma unroll
            for (int kc = 0; kc < KCU; ++kc) {
#pragma unroll
                for (int ib = 0; ib < NIB; ++ib) {
                    if (kc < KC1)
                        s[ib] = M::mma(yf[kc], xf[ib][kc], kc == 0 ? zero : s[ib]);
                    else
                        s2[ib] = M::mma(yf[kc], xf[ib][kc], kc == KC1 ? zero : s2[ib]);
                }
                if constexpr (decltype(with_z)::value) {
#pragma unroll
                    for (int f = 0; f < NZF; ++f)
                        if (f * KCU / NZF == kc) zf[f] = z_read(za, zsub, f);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // phase 2: Out += P_prev Z_prev, interleaved with the Y fragment reads of the next sub-tile
        // and the rounding of S into `pcur`
        auto phase2 = [&](auto with_pv, V8 (&pprev)[NIB][2], V8 (&pcur)[NIB][2], const int (&ya)[YQ], int ysub,
                          auto &&after_group) {
            constexpr int NPK = NIB * 8;  // packed pairs that make up P of one sub-tile
            u32x4 pk[NIB][2];
            static_for<0, NZF>([&](auto ff) {
                constexpr int f = decltype(ff)::value;
                if constexpr (decltype(with_pv)::value) {
                    const int t = f / DB, db = f % DB;
#pragma unroll
                    for (int ib = 0; ib < NIB; ++ib) acc[ib][db] = M::mma(zf[f], pprev[ib][t], acc[ib][db]);
                }
#pragma unroll
                for (int kc = 0; kc < KCU; ++kc)
                    if (kc * NZF / KCU == f) yf[kc] = y_read(ya, ysub, kc);
                if constexpr (POLY) {
                    if (f == NZF / 2) {
#pragma unroll
                        for (int ib = 0; ib < NIB; ++ib) map_scores(s[ib]);
                    }
                }
                if constexpr (DUAL) {
                    if (f == NZF / 2) {
#pragma unroll
                        for (int ib = 0; ib < NIB; ++ib) combine_scores(s[ib], s2[ib]);
                    }
                }
                if constexpr (NORM) {
                    if (f == NZF / 2) {
#pragma unroll
                        for (int ib = 0; ib < NIB; ++ib) add_scores(s[ib], rsum[ib]);
                    }
                }
                // S of this sub-tile is complete once a couple of the independent MFMAs above have
                // issued; its rounding is spread over the second half of the phase
#pragma unroll
                for (int c = 0; c < NPK; ++c) {
                    if (NZF / 2 + (c * (NZF - NZF / 2)) / NPK == f) {
                        const int ib = c / 8, t = (c / 4) % 2, w = c % 4;
                        pk[ib][t][w] = round_pack_pinned<T>(s[ib][8 * t + 2 * w], s[ib][8 * t + 2 * w + 1]);
                    }
                }
                after_group(ff);
                __builtin_amdgcn_sched_barrier(0);
            });
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib)
#pragma unroll
                for (int t = 0; t < 2; ++t) pcur[ib][t] = __builtin_bit_cast(V8, pk[ib][t]);
        };
        auto tile_body = [&](auto first) {
            constexpr bool kFirst = decltype(first)::value;
            int ya_cur[YQ], za_cur[ZQ], ya_next[YQ], za_prev[ZQ], unused_y[YQ], unused_z[ZQ];
            slot_addrs(cur_off, ya_cur, za_cur);
            slot_addrs(prev_off, unused_y, za_prev);
            slot_addrs(next_off, ya_next, unused_z);
            // first sub-tile: Z of the previous tile's second sub-tile, then Y of this tile's second
            phase1(std::integral_constant<bool, !kFirst>{}, za_prev, 1);
            phase2(std::integral_constant<bool, !kFirst>{}, pfb, pfa, ya_cur, 1, [](auto) {});
            // second sub-tile
            phase1(std::true_type{}, za_cur, 0);
            wait_tile();
            __builtin_amdgcn_s_barrier();  // tile q+1 has landed; nobody reads tile q-1 any more
            // The loads of tile q + NBUF - 1 go into the slot the barrier has just retired.  A wave
            // issues one instruction every few clocks and a load to LDS holds it for longer than
            // that, so all of them in a row would leave the matrix pipe idle: one (or a few) after
            // each group of MFMAs instead.
            {
                uint32_t so[Cfg::NT];
                tile_offsets(q + Cfg::NBUF - 1, so);
                const uint32_t yb = lds_wave + prev_off;
                phase2(std::true_type{}, pfa, pfb, ya_next, 0, [&](auto ff) {
                    static_for<0, Cfg::NT>([&](auto ii) {
                        if constexpr (decltype(ii)::value * NZF / Cfg::NT == decltype(ff)::value)
                            issue_part_at(ii, so[decltype(ii)::value], yb);
                    });
                });
            }
            advance();
            ++q;
        };
        tile_body(std::true_type{});
        while (q < n_full) tile_body(std::false_type{});
        // drain: the last sub-tile's P still has to meet its Z (second half of the previous slot)
        {
            int unused_y[YQ], za_prev[ZQ];
            slot_addrs(prev_off, unused_y, za_prev);
#pragma unroll
            for (int f = 0; f < NZF; ++f) zf[f] = z_read(za_prev, 1, f);
#pragma unroll
            for (int f = 0; f < NZF; ++f) {
                const int t = f / DB, db = f % DB;
#pragma unroll
                for (int ib = 0; ib < NIB; ++ib) acc[ib][db] = M::mma(zf[f], pfb[ib][t], acc[ib][db]);
            }
        }
    }

    // ---- chunked evaluation: Out_tile += X_tile . S with S^T[e][d] as A operand (row = output
    // column as permuted in the accumulators, k = d) and the resident X fragments as B operand.
    if (has_state) {
        // accumulator register v of lane (l32, g) is column 16 g + v of its block; MFMA row
        // m = 8a + 4g' + b of the A operand lands in register 4a + b of the lanes with g = g'
        const int e_lane = 16 * ((l32 >> 2) & 1) + 4 * (l32 >> 3) + (l32 & 3);
        // two column blocks of fragments in flight: the loads of block db+1 overlap the MFMAs of db
        V8 sf[2][KC];
        if (Cfg::kStateTransposable && p.state_transposed) {
            // From LDS, stored as S[d][e]: the fragment is a column read, eight consecutive rows d of
            // one column e per lane, i.e. the transposing read of the Z fragments with rows
            // 8g .. 8g+7 of each 16-row k chunk (the k order of the X fragments) and the same
            // lane -> column assignment as the accumulators.
            int tl[ZQ];
            {
                const int srow = 8 * g + (lam >> 2);
                const int sz = swizzle_z<CZ>(srow);
                const int zc = lam & 3, beta = (lane >> 4) & 1;
#pragma unroll
                for (int j = 0; j < ZQ; ++j) {
                    tl[j] = Cfg::SMEM_BYTES + srow * RZ + (((4 * j + 2 * (zc & 1) + beta) ^ sz) << 4) + 8 * (zc >> 1);
                    asm volatile("" : "+v"(tl[j]));  // computed here, not once per kernel
                }
            }
            auto load_block = [&](int db, V8 (&dst)[KC]) {
#pragma unroll
                for (int kc = 0; kc < KC; ++kc) {
                    const unsigned char *zp = smem + tl[db % ZQ] + (16 * kc * RZ + (db / ZQ) * (ZQ * 64));
                    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(zp));
                    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(zp + 4 * RZ));
                    dst[kc] = __builtin_bit_cast(V8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                }
            };
            load_block(0, sf[0]);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                if (db + 1 < DB) load_block(db + 1, sf[(db + 1) & 1]);
#pragma unroll
                for (int kc = 0; kc < KC; ++kc)
#pragma unroll
                    for (int ib = 0; ib < NIB; ++ib) acc[ib][db] = M::mma(sf[db & 1][kc], xf[ib][kc], acc[ib][db]);
            }
        } else if constexpr (Cfg::kStateInLds) {
            // from LDS, in the Y tile layout (row e, chunk index XOR swizzle(e))
            int sl[YQ];
            const int sw = swizzle_y<CY>(e_lane);
#pragma unroll
            for (int j = 0; j < YQ; ++j) {
                sl[j] = Cfg::SMEM_BYTES + e_lane * RY + (((2 * j + g) ^ sw) << 4);
                asm volatile("" : "+v"(sl[j]));  // computed here, not once per kernel
            }
            auto load_block = [&](int db, V8 (&dst)[KC]) {
#pragma unroll
                for (int kc = 0; kc < KC; ++kc)
                    dst[kc] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4 *>(
                                                         smem + sl[kc % YQ] + (db * 32 * RY + (kc / YQ) * (YQ * 32))));
            };
            load_block(0, sf[0]);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                if (db + 1 < DB) load_block(db + 1, sf[(db + 1) & 1]);
#pragma unroll
                for (int kc = 0; kc < KC; ++kc)
#pragma unroll
                    for (int ib = 0; ib < NIB; ++ib) acc[ib][db] = M::mma(sf[db & 1][kc], xf[ib][kc], acc[ib][db]);
            }
        } else {
            // straight from global memory: one lane offset for all fragments, column block and
            // k chunk go into the scalar offset
            const __amdgpu_buffer_rsrc_t rs =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(st), 0, DO * DC * 2, 0x00020000);
            uint32_t st_lane = (uint32_t)((e_lane * DC + 8 * g) * 2);
            asm volatile("" : "+v"(st_lane));  // keeps derived addresses from being hoisted out of the pass loop
            auto load_block = [&](int db, V8 (&dst)[KC]) {
#pragma unroll
                for (int kc = 0; kc < KC; ++kc)
                    dst[kc] = __builtin_bit_cast(
                        V8, __builtin_amdgcn_raw_buffer_load_b128(rs, st_lane, 32 * db * DC * 2 + 32 * kc, 0));
            };
            load_block(0, sf[0]);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                if (db + 1 < DB) load_block(db + 1, sf[(db + 1) & 1]);
#pragma unroll
                for (int kc = 0; kc < KC; ++kc)
#pragma unroll
                    for (int ib = 0; ib < NIB; ++ib) acc[ib][db] = M::mma(sf[db & 1][kc], xf[ib][kc], acc[ib][db]);
            }
        }
    }

    // ================= the diagonal block =================
    // Its tiles (BM / BN of them, never more than the ring holds) are all made resident first;
    // then every wave walks the 32-row sub-tiles its two row blocks touch, without barriers,
    // fetching the fragments of the next sub-tile while the MFMAs of the current one run.
    {
        static_assert(BM / BN <= Cfg::NBUF, "the diagonal block must fit in the LDS ring");
        if (n_full > 0) __builtin_amdgcn_s_barrier();  // every wave is done with the last full tile
        if constexpr (!chunked) issue_tile(q + Cfg::NBUF - 1, prev_off);  // the one tile not yet requested (if any)
        wait_vm<0>();
        __builtin_amdgcn_s_barrier();

        const int nsub = (diag_rows + 31) >> 5;  // sub-tiles with at least one valid row
        int blk_min = blk[0], blk_max = blk[0];
        if constexpr (NIB == 2) {
            blk_min = blk[0] < blk[1] ? blk[0] : blk[1];
            blk_max = blk[0] < blk[1] ? blk[1] : blk[0];
        }
        const int s_lo = upper ? blk_min : 0;
        const int s_hi = upper ? nsub - 1 : (blk_max < nsub - 1 ? blk_max : nsub - 1);

        auto load_sub = [&](int s8, V8 (&yf)[KC], V8 (&zf)[NZF]) {
            int so = cur_off + (s8 >> 1) * STAGE;
            if (so >= RING) so -= RING;
            int ya[YQ], za[ZQ];
#pragma unroll
            for (int j = 0; j < YQ; ++j) ya[j] = ylane[j] + so + (s8 & 1) * (32 * RY);
#pragma unroll
            for (int j = 0; j < ZQ; ++j) za[j] = zlane[j] + so + (s8 & 1) * (32 * RZ);
#pragma unroll
            for (int kc = 0; kc < KCU; ++kc) yf[kc] = y_read(ya, 0, kc);
#pragma unroll
            for (int f = 0; f < NZF; ++f) zf[f] = z_read(za, 0, f);
        };
        auto compute_sub = [&](int s8, const V8 (&yf)[KC], const V8 (&zf)[NZF]) {
            bool act[NIB];
            f32x16 sd[NIB], sd2[NIB];
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib) {
                act[ib] = upper ? s8 >= blk[ib] : s8 <= blk[ib];
                if (act[ib]) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) sd[ib][v] = 0.f, sd2[ib][v] = 0.f;
#pragma unroll
                    for (int kc = 0; kc < KC1; ++kc) sd[ib] = M::mma(yf[kc], xf[ib][kc], sd[ib]);
#pragma unroll
                    for (int kc = KC1; kc < KCU; ++kc) sd2[ib] = M::mma(yf[kc], xf[ib][kc], sd2[ib]);
                    if constexpr (DUAL) combine_scores(sd[ib], sd2[ib]);
                }
            }
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib) {
                if (!act[ib]) continue;
                if constexpr (POLY) map_scores(sd[ib]);  // before the mask: masked scores stay zero
                if (s8 == blk[ib]) {  // the 32 x 32 block on the diagonal itself
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int jl = 8 * (v / 4) + 4 * g + (v % 4);
                        const bool keep = upper ? l32 <= jl : l32 >= jl;
                        sd[ib][v] = keep ? sd[ib][v] : 0.f;
                    }
                }
                if constexpr (NORM) add_scores(sd[ib], rsum[ib]);
                V8 pf[2];
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int e = 0; e < 8; ++e) pf[t][e] = static_cast<T>(sd[ib][8 * t + e]);
#pragma unroll
                for (int f = 0; f < NZF; ++f) acc[ib][f % DB] = M::mma(zf[f], pf[f / DB], acc[ib][f % DB]);
            }
        };
        if (s_lo <= s_hi) {
            V8 yfa[KC], zfa[NZF], yfb[KC], zfb[NZF];
            load_sub(s_lo, yfa, zfa);
            for (int s8 = s_lo; s8 <= s_hi; s8 += 2) {
                // the scheduling barriers keep the compiler from sinking the prefetch next to its use
                if (s8 + 1 <= s_hi) load_sub(s8 + 1, yfb, zfb);
                __builtin_amdgcn_sched_barrier(0);
                compute_sub(s8, yfa, zfa);
                __builtin_amdgcn_sched_barrier(0);
                if (s8 + 1 <= s_hi) {
                    if (s8 + 2 <= s_hi) load_sub(s8 + 2, yfa, zfa);
                    __builtin_amdgcn_sched_barrier(0);
                    compute_sub(s8 + 1, yfb, zfb);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        __builtin_amdgcn_s_barrier();  // all LDS reads of the walk are done: the ring can be reused
    }

    // ---- the next row tile's first requests go out before this one's epilogue
    const int out_i0 = i0;
    const bool more = pass + 1 < n_pass;
    if constexpr (kOverlap) {
        if (more) {
            set_tile(stream_tile(pass + 1));
            ring0 = kStageSlots * STAGE;
            start_tile();
        }
    }
    // ---- epilogue.  The second product is issued as Out^T += Z^T P^T (the two register
    // operands swapped), and with the column permutation of the Z fragments acc[ib][db][v] is
    // Out[row l32 of block ib][column 32 db + 16 g + v]: 16 consecutive columns per lane.
    // They go to LDS as two 16-byte writes (the ring is idle: every wave has passed the last
    // barrier of the walk), and the tile leaves as whole rows, 16 bytes per lane.
    if constexpr (NORM) {
#pragma unroll
        for (int ib = 0; ib < NIB; ++ib) {
            const float n = rsum[ib] + __shfl_xor(rsum[ib], 32, 64) + p.eps;
            const float inv = 1.0f / n;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[ib][db][v] *= inv;
            const int row = out_i0 + blk[ib] * 32 + l32;
            if (g == 0 && row < N) p.denom[(int64_t)bh * N + row] = n;
        }
    }
    if constexpr (chunked) {
        if (p.omap) {
            // Out is the gradient with respect to y = phi(x): multiply by phi'(x), computed from y, for
            // the gradient with respect to x.  A lane holds 16 consecutive columns of one row per
            // (row block, column block).
            const T *M = static_cast<const T *>(p.omap) + b * p.ms_b + h * p.ms_h;
            const __amdgpu_buffer_rsrc_t rm = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<T *>(M), 0, (N - 1) * (int)p.ms_n * 2 + p.dout * 2, 0x00020000);
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib) {
                const int row = out_i0 + blk[ib] * 32 + l32;
#pragma unroll
                for (int db = 0; db < DB; ++db) {
#pragma unroll
                    for (int hq = 0; hq < 2; ++hq) {
                        const int col = 32 * db + 16 * g + 8 * hq;
                        const uint32_t off = (uint32_t)(row * (int)p.ms_n * 2 + col * 2) + (col < p.dout ? 0u : kOobOffset);
                        const V8 mv = __builtin_bit_cast(V8, __builtin_amdgcn_raw_buffer_load_b128(rm, off, 0, 0));
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            acc[ib][db][8 * hq + e] *= feature_slope_from_value(p.map_out, static_cast<float>(mv[e]));
                    }
                }
            }
        }
    }
    {
        constexpr int RO = Cfg::RO;
#pragma unroll
        for (int ib = 0; ib < NIB; ++ib) {
            unsigned char *rowp = smem + (blk[ib] * 32 + l32) * RO + 32 * g;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
#pragma unroll
                for (int hq = 0; hq < 2; ++hq) {
                    V8 o8;
#pragma unroll
                    for (int e = 0; e < 8; ++e) o8[e] = static_cast<T>(acc[ib][db][8 * hq + e]);
                    *reinterpret_cast<u32x4 *>(rowp + 64 * db + 16 * hq) = __builtin_bit_cast(u32x4, o8);
                }
            }
        }
        // LDS writes done, then a bare barrier: __syncthreads() would also wait for every load in
        // flight, and the next row tile's first loads are in flight here
        asm volatile("" ::: "memory");  // the compiler keeps the staging writes above, the reads below
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        constexpr int CO = DO / 8;  // 16-byte chunks per output row
        // all LDS reads first (the accumulators are dead, registers are free), then the stores:
        // read, wait, store per row would pay the LDS latency once per row
        constexpr int NOUT = BM * CO / 256;
        u32x4 val[NOUT];
#pragma unroll
        for (int u = 0; u < NOUT; ++u) {
            const int c = tid + 256 * u, r = c / CO, cc = c - r * CO;
            val[u] = *reinterpret_cast<const u32x4 *>(smem + r * RO + cc * 16);
        }
#pragma unroll
        for (int u = 0; u < NOUT; ++u) {
            const int c = tid + 256 * u, r = c / CO, cc = c - r * CO;
            const int row = out_i0 + r;
            if (row < N && cc * 8 < p.dout) *reinterpret_cast<u32x4 *>(O + (int64_t)row * p.os_n + cc * 8) = val[u];
        }
        // Every wave has read its part of the staging area (the stores above hold the values):
        // it is ring space again.  The stores themselves need not have completed.
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
    if (!more) break;
    if constexpr (!kOverlap) {
        set_tile(stream_tile(pass + 1));
        ring0 = 0;
        start_tile();
    }
    }  // pass
#else
    (void)p;
    (void)wg_index;
#endif
}

template <typename T, int DC, int DO, bool CHUNKED, int FLAGS>
__global__ __launch_bounds__(256, (FastConfig<DC, DO, CHUNKED>::kMinWavesPerSimd)) void tri_xyt_z_fast_kernel(
    const TriParams p) {
    tri_fast_body<T, DC, DO, CHUNKED, FLAGS>(p, blockIdx.x);
}

// grid y = product index
template <typename T, int DC, int DO>
__global__ __launch_bounds__(256, (FastConfig<DC, DO, false>::kMinWavesPerSimd)) void tri_xyt_z_fast_batch_kernel(
    const TriBatch b) {
    tri_fast_body<T, DC, DO, false>(b.p[blockIdx.y], blockIdx.x);
}

// Chunk-wise evaluation of up to three products of one square shape by the same workgroup, one
// after the other, for the same (head, chunk): the backward's dQ, dV and dK read the same rows
// of q, k, v and dO in different roles, so after the first product the others find them in the
// caches instead of fetching them from memory again.
template <typename T, int DC, int DO>
__global__ __launch_bounds__(256, (FastConfig<DC, DO, true>::kMinWavesPerSimd)) void tri_xyt_z_fast_chunked_batch_kernel(
    const TriBatch b, const int count) {
#pragma unroll 1
    for (int i = 0; i < count; ++i) tri_fast_body<T, DC, DO, true>(b.p[i], blockIdx.x);
}

// True when the fast kernel can take this problem: every operand 16-byte
// aligned with widths in whole chunks, rows that do not overlap, and each
// (b, h) slice addressable with 32-bit byte offsets.
inline bool fast_path_ok(const TriParams &p) {
    if (!(p.vec_x && p.vec_y && p.vec_z && p.vec_out)) return false;
    // Rows beyond N are aimed past the end of a buffer resource that covers rows 0 .. N-1 and arrive
    // as zeros: with a row stride below the width (a tensor expanded along the sequence has stride
    // 0) those offsets would fall inside it again.  Such operands take the bounds-checked kernel.
    if (p.xs_n < p.dc || p.ys_n < p.dc || p.zs_n < p.dout || p.os_n < p.dout) return false;
    const int64_t n = p.N;
    return n * p.xs_n * 2 <= kMaxFastExtent && n * p.ys_n * 2 <= kMaxFastExtent && n * p.zs_n * 2 <= kMaxFastExtent;
}

// A problem with fewer tile pairs than workgroups fit on the chip at once (256 CUs, one or two
// workgroups each) runs as single tiles, heaviest first: pairs would leave slots idle (measured
// 7-20 % faster there).  Exactly one pair per CU stays paired: every CU then has the same work
// (1-4 % faster than single tiles; also for the kernels that could run two workgroups per CU:
// fp16 B 4, H 16, N 2048, D 64 forward takes 34.0 - 34.6 us paired, 35.7 us as 512 single tiles heaviest
// first, 33.7 us with the tiles ordered so that workgroups g and g + 256, which share a CU, add up to
// equal work -- within the spread between runs, not kept --, 37.6 us with neighbours in the grid
// complementary).
constexpr int kCuCount = 256;
inline int run_single_tiles(int64_t pairs, int workgroups_per_cu) {
    return pairs < (int64_t)kCuCount * workgroups_per_cu && pairs % kCuCount != 0;
}

template <typename T, int DC, int DO, bool CHUNKED, int FLAGS>
hipError_t launch_tri_fast_variant(TriParams p, hipStream_t stream);

template <typename T, int DC, int DO>
hipError_t launch_tri_fast(const TriParams &p, hipStream_t stream) {
    if (p.state)
        return (p.denom || p.poly_on) ? hipErrorNotSupported : launch_tri_fast_variant<T, DC, DO, true, 0>(p, stream);
    if (p.map_x || p.omap) return hipErrorNotSupported;  // chunk-wise kernel only
    if (p.poly_on == 2) {  // dual-score walk: built for 32-wide outputs (the argument of the score map)
        if constexpr (DC >= 64 && DO == 32) {
            return p.denom ? hipErrorNotSupported : launch_tri_fast_variant<T, DC, DO, false, kDualFlag>(p, stream);
        } else {
            return hipErrorNotSupported;
        }
    }
    if (p.poly_on == 3) {  // dual-score walk, second operand in the last 32 columns
        if constexpr (DC >= 64 && DO == 32) {
            return p.denom ? hipErrorNotSupported
                           : launch_tri_fast_variant<T, DC, DO, false, kDualFlag | kTailFlag>(p, stream);
        } else {
            return hipErrorNotSupported;
        }
    }
    if (p.poly_on) {
        if constexpr (DC <= kPolyMaxContraction) {
            return p.denom ? launch_tri_fast_variant<T, DC, DO, false, kPolyFlag | kNormFlag>(p, stream)
                           : launch_tri_fast_variant<T, DC, DO, false, kPolyFlag>(p, stream);
        } else {
            return hipErrorNotSupported;
        }
    }
    return p.denom ? launch_tri_fast_variant<T, DC, DO, false, kNormFlag>(p, stream)
                   : launch_tri_fast_variant<T, DC, DO, false, 0>(p, stream);
}

template <typename T, int DC, int DO, bool CHUNKED, int FLAGS>
hipError_t launch_tri_fast_variant(TriParams p, hipStream_t stream) {
    using Cfg = FastConfig<DC, DO, CHUNKED>;
    if constexpr (!Cfg::kSupported) {
        return hipErrorNotSupported;
    } else {
        if (CHUNKED && p.state_transposed && !Cfg::kStateTransposable) return hipErrorNotSupported;
        p.n_tiles = (p.N + Cfg::BM - 1) / Cfg::BM;
        p.single = (!CHUNKED && run_single_tiles((int64_t)p.BH * ((p.n_tiles + 1) / 2), Cfg::kMinWavesPerSimd)) ? 1 : 0;
        const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * ((CHUNKED || p.single) ? p.n_tiles : (p.n_tiles + 1) / 2);
        if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
        constexpr auto kern = tri_xyt_z_fast_kernel<T, DC, DO, CHUNKED, FLAGS>;
        constexpr int smem = Cfg::SMEM_BYTES + (Cfg::kStateInLds ? Cfg::STATE_BYTES : 0);
        if (hipError_t e = ensure_dynamic_lds<kern>(smem)) return e;
        return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem, stream, p);
    }
}

// `count` products of the same shape (same N, B H, instantiation) in one launch.
template <typename T, int DC, int DO>
hipError_t launch_tri_fast_batch(TriBatch b, int count, hipStream_t stream) {
    using Cfg = FastConfig<DC, DO, false>;
    if constexpr (!Cfg::kSupported) {
        return hipErrorNotSupported;
    } else {
        const int n_tiles = (b.p[0].N + Cfg::BM - 1) / Cfg::BM;
        const int single = run_single_tiles((int64_t)b.p[0].BH * ((n_tiles + 1) / 2), Cfg::kMinWavesPerSimd);
        for (int i = 0; i < count; ++i) b.p[i].n_tiles = n_tiles, b.p[i].single = single, b.p[i].state = nullptr;
        const int64_t grid = (int64_t)8 * ((b.p[0].BH + 7) / 8) * (single ? n_tiles : (n_tiles + 1) / 2);
        if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
        constexpr auto kern = tri_xyt_z_fast_batch_kernel<T, DC, DO>;
        if (hipError_t e = ensure_dynamic_lds<kern>(Cfg::SMEM_BYTES)) return e;
        return launch_kernel<kern>(dim3((unsigned)grid, (unsigned)count), dim3(256), Cfg::SMEM_BYTES, stream, b);
    }
}

// `count` chunk-wise products of one square shape, every TriParams with its state set, evaluated
// by the same workgroups in sequence (see tri_xyt_z_fast_chunked_batch_kernel).
template <typename T, int DC, int DO>
hipError_t launch_tri_fast_chunked_batch(TriBatch b, int count, hipStream_t stream) {
    using Cfg = FastConfig<DC, DO, true>;
    if constexpr (!Cfg::kSupported || DC != DO) {
        return hipErrorNotSupported;
    } else {
        const int n_tiles = (b.p[0].N + Cfg::BM - 1) / Cfg::BM;
        for (int i = 0; i < count; ++i) {
            if (!b.p[i].state || (b.p[i].state_transposed && !Cfg::kStateTransposable)) return hipErrorNotSupported;
            b.p[i].n_tiles = n_tiles, b.p[i].single = 0;
        }
        const int64_t grid = (int64_t)8 * ((b.p[0].BH + 7) / 8) * n_tiles;
        if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
        constexpr auto kern = tri_xyt_z_fast_chunked_batch_kernel<T, DC, DO>;
        constexpr int smem = Cfg::SMEM_BYTES + (Cfg::kStateInLds ? Cfg::STATE_BYTES : 0);
        if (hipError_t e = ensure_dynamic_lds<kern>(smem)) return e;
        return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem, stream, b, count);
    }
}

}  // namespace fla

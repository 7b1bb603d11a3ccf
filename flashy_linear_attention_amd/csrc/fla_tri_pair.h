// Two masked products that stream the same tiles, in one kernel:
//
//     OutA = upper(XA YA^T) YB        OutB = upper(XB YB^T) YA
//
// which is the backward's dV = upper(K Q^T) dO and dK = upper(V dO^T) Q (XA = K, XB = V, YA = Q,
// YB = dO; the reference forms both in one loop over the query blocks as well,
// flashlinear/kernels/linear_attn_kernels.py:160-227).  A workgroup owns BM rows of K and V --
// their MFMA operand fragments and the fp32 accumulators of its dV and dK rows stay in registers
// for the whole walk -- and the (Q, dO) tiles are brought to LDS once for both products: each tile
// is read along its rows as the Y operand of one product's scores and down its columns as the Z
// operand of the other product's second contraction.  One layout serves both kinds of read
// (walk_swizzle, fla_chunk_walk.h).  Everything else is the scheme of fla_tri_fast.h: LDS-DMA ring,
// S^T accumulators chained into the second MFMA from registers, a software-pipelined walk over the
// tiles that lie wholly inside the mask, then the diagonal block.
//
// Built for equal padded head dims: 64 rows per wave up to D = 64 (four sets of operand fragments
// and two sets of accumulators need about 490 registers there, one wave per SIMD), 32 rows per
// wave at D = 128 (the two sets of accumulators alone are 128 registers per 32 rows).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fla_chunk_walk.h"
#include "fla_tri_fast.h"

namespace fla {

struct TriPairParams {
    const void *xa, *xb;  // resident rows: X of product A (k), X of product B (v)
    const void *ya, *yb;  // streamed rows: Y of A and Z of B (q); Y of B and Z of A (grad of the output)
    void *oa, *ob;        // OutA (dv), OutB (dk)
    int64_t xas_b, xas_h, xas_n, xbs_b, xbs_h, xbs_n;  // element strides; the innermost stride is 1
    int64_t yas_b, yas_h, yas_n, ybs_b, ybs_h, ybs_n;
    int64_t oas_b, oas_h, oas_n, obs_b, obs_h, obs_n;
    int32_t H, N, BH;
    int32_t wa, wb;   // true widths: wa of xa, ya, ob (contraction of A, output of B); wb of xb, yb, oa
    int32_t n_tiles;  // ceil(N / BM), filled by the launcher
    int32_t single;   // one row tile per workgroup instead of a balanced pair (launcher's choice)
};

template <int D>
struct PairConfig {
    static constexpr int NIB = D <= 64 ? 2 : 1;  // 32-row blocks per wave
    static constexpr int MW = 32 * NIB, NW = 4, BM = MW * NW, BN = 64;
    static constexpr int RB = D * 2, CR = D / 8;  // bytes and 16-byte chunks per tile row
    static constexpr int TILE = BN * RB;          // one operand tile
    static constexpr int STAGE = 2 * TILE;        // YA tile, then YB tile
    static constexpr int kMaxSlots = (160 * 1024) / STAGE;
    static constexpr int NBUF = kMaxSlots >= 6 ? 6 : kMaxSlots;
    static constexpr int SMEM_BYTES = NBUF * STAGE;
    static constexpr int NI = TILE / 4096;  // wave-level 1 KiB loads per operand tile and wave
    static constexpr int NT = 2 * NI;       // buffer loads per wave and tile pair
    static constexpr int RPI = 1024 / RB;   // rows one such load covers
    static constexpr int RO = D * 2 + 16;   // output staging: BM rows, 16 bytes of padding each
    static_assert(D == 32 || D == 64 || D == 128, "built for padded head dims 32, 64 and 128");
    static_assert(BM / BN <= NBUF - 1, "the diagonal block must fit in the ring");
    static_assert(BM * RO <= SMEM_BYTES, "output staging must fit in the ring");
    static_assert(NI == 1 || (4 * RPI) % 16 == 0, "the swizzle must not depend on the load index");
};

template <typename T, int D>
__global__ __launch_bounds__(256, 1) void tri_pair_upper_kernel(const TriPairParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    using Cfg = PairConfig<D>;
    using M = Mma<T>;
    using V8 = typename M::V8;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NIB = Cfg::NIB, NBLK = BM / 32;
    constexpr int KC = D / 16, DB = D / 32, NZF = 2 * DB;
    constexpr int RB = Cfg::RB, CR = Cfg::CR, TILE = Cfg::TILE, STAGE = Cfg::STAGE, NI = Cfg::NI;
    constexpr int RING = Cfg::NBUF * STAGE;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, g = lane >> 5, lam = lane & 15;

    // workgroup -> (head, row tiles): heads to XCDs by id % 8, as in fla_tri_fast.h
    const int wg = blockIdx.x, xcd = wg & 7, slot = wg >> 3;
    const bool single = p.single != 0;
    const int n_pairs = single ? p.n_tiles : (p.n_tiles + 1) >> 1;
    const int n_hl = (p.BH + 7) >> 3;
    const int hl = single ? slot % n_hl : slot / n_pairs;
    const int rank = single ? slot / n_hl : slot - hl * n_pairs;
    const int bh = hl * 8 + xcd;
    if (bh >= p.BH) return;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N;
    const T *XA = static_cast<const T *>(p.xa) + b * p.xas_b + h * p.xas_h;
    const T *XB = static_cast<const T *>(p.xb) + b * p.xbs_b + h * p.xbs_h;
    const T *YA = static_cast<const T *>(p.ya) + b * p.yas_b + h * p.yas_h;
    const T *YB = static_cast<const T *>(p.yb) + b * p.ybs_b + h * p.ybs_h;
    T *OA = static_cast<T *>(p.oa) + b * p.oas_b + h * p.oas_h;
    T *OB = static_cast<T *>(p.ob) + b * p.obs_b + h * p.obs_h;
    const int xas2 = (int)p.xas_n * 2, xbs2 = (int)p.xbs_n * 2, yas2 = (int)p.yas_n * 2, ybs2 = (int)p.ybs_n * 2;
    // raw buffer resources covering exactly the valid rows of this (b, h): rows beyond N and chunks
    // beyond the true width are aimed outside and arrive as zeros
    const __amdgpu_buffer_rsrc_t rxa =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(XA), 0, (N - 1) * xas2 + p.wa * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rxb =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(XB), 0, (N - 1) * xbs2 + p.wb * 2, 0x00020000);
    const u32x4 rya = make_rsrc(YA, (uint32_t)((N - 1) * yas2 + p.wa * 2));
    const u32x4 ryb = make_rsrc(YB, (uint32_t)((N - 1) * ybs2 + p.wb * 2));

    // with two row blocks per wave, wave w owns blocks w and 7 - w of the tile: equal work on the diagonal block
    const int blk[2] = {wave, NBLK - 1 - wave};  // (the second entry is unused with one block per wave)

    // ---- the row tiles of this workgroup: pairs (t, T-1-t) have equal work under the mask; unpaired
    // tiles go heaviest first (under the upper mask that is tile 0)
    auto stream_tile = [&](int pass) { return single ? rank : (pass == 0 ? rank : p.n_tiles - 1 - rank); };
    const int n_pass = (single || rank == p.n_tiles - 1 - rank) ? 1 : 2;
    int i0 = 0, diag_rows = 0, n_full = 0, n_seq = 0;
    auto set_tile = [&](int t) {
        i0 = t * BM;
        diag_rows = (N - i0 < BM) ? (N - i0) : BM;
        const int rest = N - (i0 + BM);
        n_full = rest > 0 ? (rest + BN - 1) / BN : 0;
        n_seq = n_full + (diag_rows + BN - 1) / BN;
    };
    // tile q of the sequence: the tiles behind the diagonal block first, then the block's own
    auto tile_row0 = [&](int q) { return q < n_full ? i0 + BM + q * BN : i0 + (q - n_full) * BN; };

    // ---- HBM -> LDS.  Load u of a wave covers rows u * 4 RPI + wave * RPI + lane / CR of a tile; the
    // lane fetches the chunk that belongs at its place under the swizzle.
    uint32_t dma_a, dma_b;
    {
        const int row = wave * Cfg::RPI + lane / CR;
        const int c = (lane % CR) ^ walk_swizzle<CR>(row);
        dma_a = (uint32_t)(row * yas2 + c * 16) + (c * 8 < p.wa ? 0u : kOobOffset);
        dma_b = (uint32_t)(row * ybs2 + c * 16) + (c * 8 < p.wb ? 0u : kOobOffset);
    }
    const uint32_t lds_wave = lds0 + wave * 1024;
    auto tile_offsets = [&](int q, uint32_t (&so)[Cfg::NT]) {
        const bool exists = q < n_seq;
        const int row0 = tile_row0(q);
        static_for<0, Cfg::NT>([&](auto ii) {
            constexpr int I = decltype(ii)::value;
            so[I] = !exists ? kOobOffset
                            : I < NI ? (uint32_t)((row0 + I * 4 * Cfg::RPI) * yas2)
                                     : (uint32_t)((row0 + (I - NI) * 4 * Cfg::RPI) * ybs2);
        });
    };
    auto issue_part_at = [&](auto ii, uint32_t soffset, uint32_t base) {
        constexpr int I = decltype(ii)::value;
        if constexpr (I < NI)
            dma_16B_per_lane<I * 4096>(rya, base, dma_a, soffset);
        else
            dma_16B_per_lane<TILE + (I - NI) * 4096>(ryb, base, dma_b, soffset);
    };
    auto issue_tile = [&](int q, int slot_off) {
        uint32_t so[Cfg::NT];
        tile_offsets(q, so);
        static_for<0, Cfg::NT>([&](auto ii) { issue_part_at(ii, so[decltype(ii)::value], lds_wave + slot_off); });
    };
    auto next_slot = [](int off) { return off + STAGE == RING ? 0 : off + STAGE; };
    // a tile has landed once at most the NBUF - 3 tiles issued after it are still in flight
    auto wait_tile = [&]() {
        static_assert((Cfg::NBUF - 3) * Cfg::NT < 64, "vmcnt is a 6-bit field");
        wait_vm<(Cfg::NBUF - 3) * Cfg::NT>();
    };

    // ---- LDS read offsets inside a stage (bytes; the YB tile sits TILE behind the YA tile)
    int rowlane[KC];              // row read of row l32: chunk 2 kc + g under the swizzle
    int col_lo[DB], col_hi[DB];   // column read (transposing): rows 4 g + lam / 4 and 8 more, columns of block db
    {
        const int sy = walk_swizzle<CR>(l32);
#pragma unroll
        for (int kc = 0; kc < KC; ++kc) rowlane[kc] = l32 * RB + (((2 * kc + g) ^ sy) << 4);
        // (the swizzle repeats every 16 rows: sub-tiles and their halves start at multiples of 16, so the
        // lane's part is the same for all of them; rows r and r + 8 differ)
        const int zrow = 4 * g + (lam >> 2), zc = lam & 3, beta = (lane >> 4) & 1;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const int ch = 4 * db + 2 * (zc & 1) + beta;
            col_lo[db] = zrow * RB + ((ch ^ walk_swizzle<CR>(zrow)) << 4) + 8 * (zc >> 1);
            col_hi[db] = (zrow + 8) * RB + ((ch ^ walk_swizzle<CR>(zrow + 8)) << 4) + 8 * (zc >> 1);
        }
    }
    // operand `which` (0: YA tile, 1: YB tile) of the stage at byte offset `so`
    auto row_read = [&](int so, int which, int sub, int kc) -> V8 {
        const unsigned char *ptr = smem + so + which * TILE + sub * 32 * RB + rowlane[kc];
        return __builtin_bit_cast(V8, *reinterpret_cast<const u32x4 *>(ptr));
    };
    // fragment f = (t, db): rows 16 t + {4g .. 4g+3, 8+4g ..} of sub-tile `sub`, columns of block db
    auto col_read = [&](int so, int which, int sub, int f) -> V8 {
        const int t = f / DB, db = f % DB;
        const unsigned char *zp = smem + so + which * TILE + (sub * 32 + 16 * t) * RB;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(zp + col_lo[db]));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(zp + col_hi[db]));
        return __builtin_bit_cast(V8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    for (int pass = 0; pass < n_pass; ++pass) {
        set_tile(stream_tile(pass));
        // ---- first requests: tile 0, the resident X fragments, tiles up to NBUF - 3
        issue_tile(0, 0);
        V8 xf[2][NIB][KC];  // [product][row block][k chunk]
#pragma unroll
        for (int ib = 0; ib < NIB; ++ib) {
            const int row = i0 + blk[ib] * 32 + l32;
#pragma unroll
            for (int kc = 0; kc < KC; ++kc) {
                const int col = kc * 16 + 8 * g;
                const uint32_t oa = (uint32_t)(row * xas2 + col * 2) + (col < p.wa ? 0u : kOobOffset);
                const uint32_t ob = (uint32_t)(row * xbs2 + col * 2) + (col < p.wb ? 0u : kOobOffset);
                xf[0][ib][kc] = __builtin_bit_cast(V8, __builtin_amdgcn_raw_buffer_load_b128(rxa, oa, 0, 0));
                xf[1][ib][kc] = __builtin_bit_cast(V8, __builtin_amdgcn_raw_buffer_load_b128(rxb, ob, 0, 0));
            }
        }
        static_for<1, Cfg::NBUF - 2>([&](auto qq) { issue_tile(decltype(qq)::value, decltype(qq)::value * STAGE); });
        wait_tile();
        __builtin_amdgcn_s_barrier();  // tile 0 and the X fragments have landed
        issue_tile(Cfg::NBUF - 2, (Cfg::NBUF - 2) * STAGE);

        f32x16 acc[2][NIB][DB];  // [product][row block][32-column block of the output]
#pragma unroll
        for (int pr = 0; pr < 2; ++pr)
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib)
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[pr][ib][db][v] = 0.f;

        int prev_off = (Cfg::NBUF - 1) * STAGE, cur_off = 0, next_off = STAGE;
        auto advance = [&]() {
            prev_off = cur_off;
            cur_off = next_off;
            next_off = next_slot(next_off);
        };
        int q = 0;

        // ================= tiles wholly inside the mask: pipelined, no masking =================
        // Per 32-row sub-tile s of (YA, YB):
        //   phase 1:  S_A = YA_s XA^T, S_B = YB_s XB^T        | column fragments of sub-tile s-1
        //   phase 2:  OutA += P_A(s-1) YB(s-1), OutB += P_B(s-1) YA(s-1)
        //                                                      | row fragments of s+1, rounding of S(s)
        if (n_full > 0) {
            V8 yf[2][KC], zf[2][NZF], pfa[2][NIB][2], pfb[2][NIB][2];
            f32x16 s[2][NIB];
            const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int pr = 0; pr < 2; ++pr)
#pragma unroll
                for (int kc = 0; kc < KC; ++kc) yf[pr][kc] = row_read(cur_off, pr, 0, kc);

            auto phase1 = [&](auto with_z, int zoff, int zsub) {
#pragma unroll
                for (int kc = 0; kc < KC; ++kc) {
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr)
#pragma unroll
                        for (int ib = 0; ib < NIB; ++ib)
                            s[pr][ib] = M::mma(yf[pr][kc], xf[pr][ib][kc], kc == 0 ? zero : s[pr][ib]);
                    if constexpr (decltype(with_z)::value) {
                        // Z of product A is the YB tile, Z of product B the YA tile
#pragma unroll
                        for (int f = 0; f < NZF; ++f)
                            if (f * KC / NZF == kc) {
                                zf[0][f] = col_read(zoff, 1, zsub, f);
                                zf[1][f] = col_read(zoff, 0, zsub, f);
                            }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            auto phase2 = [&](auto with_pv, V8 (&pprev)[2][NIB][2], V8 (&pcur)[2][NIB][2], int yoff, int ysub,
                              auto &&after_group) {
                constexpr int NPK = 2 * NIB * 8;  // packed pairs that make up P of one sub-tile, both products
                u32x4 pk[2][NIB][2];
                static_for<0, NZF>([&](auto ff) {
                    constexpr int f = decltype(ff)::value;
                    if constexpr (decltype(with_pv)::value) {
                        const int t = f / DB, db = f % DB;
#pragma unroll
                        for (int pr = 0; pr < 2; ++pr)
#pragma unroll
                            for (int ib = 0; ib < NIB; ++ib)
                                acc[pr][ib][db] = M::mma(zf[pr][f], pprev[pr][ib][t], acc[pr][ib][db]);
                    }
#pragma unroll
                    for (int kc = 0; kc < KC; ++kc)
                        if (kc * NZF / KC == f) {
                            yf[0][kc] = row_read(yoff, 0, ysub, kc);
                            yf[1][kc] = row_read(yoff, 1, ysub, kc);
                        }
                    // S of this sub-tile is complete once the first MFMAs above have issued; its
                    // rounding is spread over the groups of the phase
#pragma unroll
                    for (int c = 0; c < NPK; ++c) {
                        if ((c * NZF) / NPK == f) {
                            const int pr = c / (NIB * 8), ib = (c / 8) % NIB, t = (c / 4) % 2, w = c % 4;
                            pk[pr][ib][t][w] =
                                round_pack_pinned<T>(s[pr][ib][8 * t + 2 * w], s[pr][ib][8 * t + 2 * w + 1]);
                        }
                    }
                    after_group(ff);
                    __builtin_amdgcn_sched_barrier(0);
                });
#pragma unroll
                for (int pr = 0; pr < 2; ++pr)
#pragma unroll
                    for (int ib = 0; ib < NIB; ++ib)
#pragma unroll
                        for (int t = 0; t < 2; ++t) pcur[pr][ib][t] = __builtin_bit_cast(V8, pk[pr][ib][t]);
            };
            auto tile_body = [&](auto first) {
                constexpr bool kFirst = decltype(first)::value;
                // first sub-tile: Z of the previous tile's second sub-tile, then Y of this tile's second
                phase1(std::integral_constant<bool, !kFirst>{}, prev_off, 1);
                phase2(std::integral_constant<bool, !kFirst>{}, pfb, pfa, cur_off, 1, [](auto) {});
                // second sub-tile
                phase1(std::true_type{}, cur_off, 0);
                wait_tile();
                __builtin_amdgcn_s_barrier();  // tile q + 1 has landed; nobody reads tile q - 1 any more
                {
                    // the loads of tile q + NBUF - 1 go into the slot just retired, one per group of MFMAs
                    uint32_t so[Cfg::NT];
                    tile_offsets(q + Cfg::NBUF - 1, so);
                    const uint32_t base = lds_wave + prev_off;
                    phase2(std::true_type{}, pfa, pfb, next_off, 0, [&](auto ff) {
                        static_for<0, Cfg::NT>([&](auto ii) {
                            if constexpr (decltype(ii)::value * NZF / Cfg::NT == decltype(ff)::value)
                                issue_part_at(ii, so[decltype(ii)::value], base);
                        });
                    });
                }
                advance();
                ++q;
            };
            tile_body(std::true_type{});
            while (q < n_full) tile_body(std::false_type{});
            // drain: the last sub-tile's P still has to meet its Z (second half of the previous slot)
#pragma unroll
            for (int f = 0; f < NZF; ++f) {
                zf[0][f] = col_read(prev_off, 1, 1, f);
                zf[1][f] = col_read(prev_off, 0, 1, f);
            }
#pragma unroll
            for (int f = 0; f < NZF; ++f) {
                const int t = f / DB, db = f % DB;
#pragma unroll
                for (int pr = 0; pr < 2; ++pr)
#pragma unroll
                    for (int ib = 0; ib < NIB; ++ib) acc[pr][ib][db] = M::mma(zf[pr][f], pfb[pr][ib][t], acc[pr][ib][db]);
            }
        }

        // ================= the diagonal block =================
        {
            if (n_full > 0) __builtin_amdgcn_s_barrier();  // every wave is done with the last full tile
            issue_tile(q + Cfg::NBUF - 1, prev_off);        // the one tile not yet requested (if any)
            wait_vm<0>();
            __builtin_amdgcn_s_barrier();

            const int nsub = (diag_rows + 31) >> 5;  // sub-tiles with at least one valid row
            const int s_lo = (NIB == 2 && blk[1] < blk[0]) ? blk[1] : blk[0], s_hi = nsub - 1;
            auto sub_off = [&](int s8) {
                int so = cur_off + (s8 >> 1) * STAGE;
                return so >= RING ? so - RING : so;
            };
            auto load_sub = [&](int s8, V8 (&yf)[2][KC], V8 (&zf)[2][NZF]) {
                const int so = sub_off(s8);
#pragma unroll
                for (int kc = 0; kc < KC; ++kc) {
                    yf[0][kc] = row_read(so, 0, s8 & 1, kc);
                    yf[1][kc] = row_read(so, 1, s8 & 1, kc);
                }
#pragma unroll
                for (int f = 0; f < NZF; ++f) {
                    zf[0][f] = col_read(so, 1, s8 & 1, f);
                    zf[1][f] = col_read(so, 0, s8 & 1, f);
                }
            };
            auto compute_sub = [&](int s8, const V8 (&yf)[2][KC], const V8 (&zf)[2][NZF]) {
                // lowest Y row (within the sub-tile) a lane keeps: its own X row on the diagonal block, any row behind it
                int bound[NIB];
#pragma unroll
                for (int ib = 0; ib < NIB; ++ib) {
                    bound[ib] = s8 == blk[ib] ? l32 : -1;
                    asm volatile("" : "+v"(bound[ib]));  // (a per-lane value: keeps the selects from becoming a branch)
                }
#pragma unroll
                for (int ib = 0; ib < NIB; ++ib) {
                    if (s8 < blk[ib]) continue;  // wholly masked for this row block
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr) {
                        f32x16 sd;
#pragma unroll
                        for (int v = 0; v < 16; ++v) sd[v] = 0.f;
#pragma unroll
                        for (int kc = 0; kc < KC; ++kc) sd = M::mma(yf[pr][kc], xf[pr][ib][kc], sd);
                        // The 32 x 32 block on the diagonal keeps X row <= Y row.  Done with selects on a
                        // per-lane bound, not under a branch: the compiler was seen to leave out the wait
                        // states between the last MFMA above and the first read of its result on the path
                        // that jumps over a masked block (wrong values, no error).
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int jl = 8 * (v / 4) + 4 * g + (v % 4);
                            sd[v] = jl >= bound[ib] ? sd[v] : 0.f;
                        }
                        V8 pf[2];
#pragma unroll
                        for (int t = 0; t < 2; ++t)
#pragma unroll
                            for (int e = 0; e < 8; ++e) pf[t][e] = static_cast<T>(sd[8 * t + e]);
#pragma unroll
                        for (int f = 0; f < NZF; ++f)
                            acc[pr][ib][f % DB] = M::mma(zf[pr][f], pf[f / DB], acc[pr][ib][f % DB]);
                    }
                }
            };
            for (int s8 = s_lo; s8 <= s_hi; ++s8) {
                V8 yfd[2][KC], zfd[2][NZF];
                load_sub(s8, yfd, zfd);
                compute_sub(s8, yfd, zfd);
            }
            __builtin_amdgcn_s_barrier();  // all LDS reads of the walk are done: the ring can be reused
        }

        // ---- epilogue, one result after the other: acc[pr][ib][db][v] is Out[row l32 of block ib][column
        // 32 db + 16 g + v]; the tile is staged in LDS and leaves as whole rows, 16 bytes per lane
        static_for<0, 2>([&](auto prr) {
            constexpr int pr = decltype(prr)::value;
            constexpr int RO = Cfg::RO;
            T *O = pr == 0 ? OA : OB;
            const int64_t os_n = pr == 0 ? p.oas_n : p.obs_n;
            const int width = pr == 0 ? p.wb : p.wa;
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib) {
                unsigned char *rowp = smem + (blk[ib] * 32 + l32) * RO + 32 * g;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int hq = 0; hq < 2; ++hq) {
                        V8 o8;
#pragma unroll
                        for (int e = 0; e < 8; ++e) o8[e] = static_cast<T>(acc[pr][ib][db][8 * hq + e]);
                        *reinterpret_cast<u32x4 *>(rowp + 64 * db + 16 * hq) = __builtin_bit_cast(u32x4, o8);
                    }
            }
            __syncthreads();
            constexpr int CO = D / 8, NOUT = BM * CO / 256;
            u32x4 val[NOUT];
#pragma unroll
            for (int u = 0; u < NOUT; ++u) {
                const int c = tid + 256 * u, r = c / CO, cc = c - r * CO;
                val[u] = *reinterpret_cast<const u32x4 *>(smem + r * RO + cc * 16);
            }
#pragma unroll
            for (int u = 0; u < NOUT; ++u) {
                const int c = tid + 256 * u, r = c / CO, cc = c - r * CO;
                const int row = i0 + r;
                if (row < N && cc * 8 < width) *reinterpret_cast<u32x4 *>(O + (int64_t)row * os_n + cc * 8) = val[u];
            }
            __syncthreads();  // the staging area is free again (for the other result, or the next row tile's ring)
        });
    }  // pass
#else
    (void)p;
#endif
}

// OutA = upper(XA YA^T) YB and OutB = upper(XB YB^T) YA for equal padded head dims D <= 128, from the two
// products' own parameter sets: a = (x: XA, y: YA, z: YB, out: OutA), b = (x: XB, y: YB, z: YA, out: OutB).
template <typename T, int D>
hipError_t launch_tri_pair(const TriParams &a, const TriParams &b, hipStream_t stream) {
    using Cfg = PairConfig<D>;
    if (!a.upper || !b.upper || a.y != b.z || a.z != b.y || a.N != b.N || a.BH != b.BH || a.H != b.H ||
        a.dc != b.dout || a.dout != b.dc || a.dc > D || a.dout > D)
        return hipErrorInvalidValue;
    TriPairParams p;
    p.xa = a.x, p.xb = b.x, p.ya = a.y, p.yb = b.y, p.oa = a.out, p.ob = b.out;
    p.xas_b = a.xs_b, p.xas_h = a.xs_h, p.xas_n = a.xs_n, p.xbs_b = b.xs_b, p.xbs_h = b.xs_h, p.xbs_n = b.xs_n;
    p.yas_b = a.ys_b, p.yas_h = a.ys_h, p.yas_n = a.ys_n, p.ybs_b = b.ys_b, p.ybs_h = b.ys_h, p.ybs_n = b.ys_n;
    p.oas_b = a.os_b, p.oas_h = a.os_h, p.oas_n = a.os_n, p.obs_b = b.os_b, p.obs_h = b.os_h, p.obs_n = b.os_n;
    p.H = a.H, p.N = a.N, p.BH = a.BH, p.wa = a.dc, p.wb = b.dc;
    p.n_tiles = (p.N + Cfg::BM - 1) / Cfg::BM;
    p.single = run_single_tiles((int64_t)p.BH * ((p.n_tiles + 1) / 2), 1) ? 1 : 0;
    const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * (p.single ? p.n_tiles : (p.n_tiles + 1) / 2);
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    constexpr auto kern = tri_pair_upper_kernel<T, D>;
    if (hipError_t e = ensure_dynamic_lds<kern>(Cfg::SMEM_BYTES)) return e;
    return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), Cfg::SMEM_BYTES, stream, p);
}

}  // namespace fla

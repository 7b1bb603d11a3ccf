// Chunk-wise causal linear attention with the running state kept inside the kernel, for equal
// padded head dims D = 32, 64 or 128 (shapes bound by memory traffic, not by the matrix units).
//
// The chunk-wise evaluation of fla_chunk_state.h / fla_tri_fast.h computes every per-chunk
// state, writes it in fp32, scans it, writes the running sums in 16 bit and reads them back in
// each consumer, and its backward reads q, k, v and dO once per product.  Here a workgroup walks
// a *segment* of consecutive chunks in sequence order and carries the running state
//
//     S = sum over the chunks before of K_c^T V_c      (forward, lower mask: ascending walk)
//     R = sum over the chunks after  of Q_c^T dO_c     (backward, upper mask: descending walk)
//
// in fp32 accumulators; per chunk it is rounded once to the storage type (as before) into LDS,
// where the MFMAs of the state products read it.  Every operand tile of a chunk is brought to
// LDS once and serves all products of that chunk:
//
//   forward   O_c  = lower(Q_c K_c^T) V_c   + Q_c S          then S += K_c^T V_c
//   backward  dQ_c = lower(dO_c V_c^T) K_c  + dO_c S_c^T
//             dV_c = upper(K_c Q_c^T) dO_c  + K_c R
//             dK_c = upper(V_c dO_c^T) Q_c  + V_c R^T        then R += Q_c^T dO_c
//
// Segments make the walk parallel: a first kernel adds up K^T V (Q^T dO) over segments, a small
// one turns the totals into each segment's entry state (exclusive prefix / suffix sums), and
// each walking workgroup starts from its segment's entry state.  No fp32 per-chunk state ever
// goes to memory.
//
//   D <= 64: 128-row chunks, two workgroups per CU.  ONE backward kernel (walk_bwd_kernel)
//            computes dQ, dV and dK of a chunk from one set of tiles; dQ's state -- the sum of
//            K^T V over the chunks BEFORE -- is obtained going backwards, by subtracting every
//            chunk's K^T V from the forward state at the segment's end, so forward hands over
//            only its segments' fp32 entry states and the state after the last chunk.  (With
//            the normaliser, whose vectors take the LDS a second state copy would need, forward
//            saves the 16-bit state at the entry of every chunk instead.)
//   D = 128: tiles and state must share the 160 KiB of LDS: 64-row chunks, one workgroup per CU
//            with two sets of tiles (the next chunk's loads are in flight while this one is
//            multiplied).  A saved per-chunk state would cost as much traffic as an operand, so
//            forward hands over the same fp32 states, and backward is ONE reverse walk as well
//            (walk_bwd_rev_kernel), with dQ's state by the same subtraction.  Without forward's
//            states, and with the normaliser, backward is split instead: dQ is the forward walk over
//            (dO, V, K), whose states V^T K start from the transposed entry states, and
//            walk_dkdv_kernel is the reverse walk for dV and dK.
//
// Options of the walks: an element-wise feature map applied to q, k as they are loaded, with its
// slope multiplied into dQ, dK (WalkParams::fmap); the normaliser of linear attention and its
// gradient terms as rank-one additions to the products (WalkParams::denom ...); at D = 128,
// operands of at most 64 true columns on one side without the MFMAs on their padding (WalkExt), and
// a result added to what its place in memory holds (WalkParams::accumulate) -- both for a wide
// q / k evaluated as two 128-column halves.
//
// Scheduling.  With one wave per SIMD nothing hides the latency of an LDS read but the wave's own
// instruction order, and the compiler, short of registers, moves every operand read down to the
// MFMA that uses it.  The products therefore name their order themselves (walk_pipe: fragment
// j + 4 is read before fragment j is used, kept in place by scheduling barriers), the state
// product's MFMAs go between the score MFMAs of the first block (D = 128), running sums that only
// MFMAs touch live in accumulation registers (Mma::mma_acc), and code for feature maps is compiled
// only into the instantiations that use it.
//
// Layout.  An operand tile is C rows x D 16-bit values, row-major, the 16-byte chunk index of
// a row XORed with walk_swizzle(row) -- one layout, free of bank conflicts for the 16-byte row
// reads (MFMA operands with k along the row) and for the transposing column reads (k down the rows).  A wave
// owns one 32-row block of the chunk as the "X rows" of every product (and, at D = 128, one half
// of the output columns; the two waves of a row block then form the same scores); the MFMA
// operand chaining is that of the other kernels: S^T = Y X^T leaves a lane holding one X row
// and eight-row groups of Y rows, which is the B operand of Out^T += Z^T P^T.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fla_launch.h"
#include "fla_tri_fast.h"

namespace fla {

// rows per chunk of the walk kernels: 128, or 64 at D = 128 (tiles and state must share the LDS)
constexpr int walk_rows(int D) { return D <= 64 ? 128 : 64; }

struct WalkParams {
    const void *q, *k, *v, *go;  // operands (go: backward only); (B, H, N, D)
    void *o, *dq, *dk, *dv;      // results (forward: o; backward: dq, dk, dv)
    int64_t qs_b, qs_h, qs_n, ks_b, ks_h, ks_n, vs_b, vs_h, vs_n, gs_b, gs_h, gs_n;
    int64_t os_b, os_h, os_n, dqs_b, dqs_h, dqs_n, dks_b, dks_h, dks_n, dvs_b, dvs_h, dvs_n;
    int32_t H, N, BH, wqk, wv;   // true widths of q/k and of v (<= D)
    int32_t n_chunks;            // ceil(N / rows per chunk)
    int32_t seg_chunks, n_seg;   // chunks per segment, segments per (b, h)
    // entry state of every segment, fp32 [BH][n_seg][D (q/k index)][D (v index)]: sum of K^T V over
    // the segments before (forward) / of Q^T dO over the segments after (backward); null when
    // there is a single segment (entry state zero).  init_transposed: the buffer holds the
    // transposed matrices ([v index][q/k index]).
    const float *init;
    int32_t init_transposed;
    // forward: where the 16-bit state at the entry of every chunk goes, [BH][n_chunks][D][D]
    // ([q/k index][v index]), or null; backward: the same buffer, read for dQ
    void *saved;
    // Feature map (fla_feature.h), 0: none.  Forward: q holds the argument xq of the map phi; the Q
    // tile is mapped in LDS as it lands and phi(xq) is written to qmap_out (q's shape, element
    // strides qo_*); k already holds phi(xk) (written by the totals kernel).  Backward: q and k
    // hold phi(xq), phi(xk), and dQ, dK are multiplied by the slope of phi, computed from those
    // values in the LDS tiles, before they are rounded and stored.
    int32_t fmap;
    void *qmap_out;
    int64_t qo_b, qo_h, qo_n;
    // walk_fwd_kernel run as the dQ walk of the split backward (q <- dO, k <- V, v <- K, o <- dQ) with
    // a feature map: slope_y holds phi(xq) (o's shape, element strides sy_*) and the result is
    // multiplied by the slope of phi computed from it; null: none.
    const void *slope_y;
    int64_t sy_b, sy_h, sy_n;
    // The normaliser n_i = q_i . (k_0 + ... + k_i) + eps fused into the walks (null pointers: off).
    // Forward (denom, zc): n_i = sum of row i's masked scores + q_i . zc_c; the result is divided by
    // n_i and n goes to denom.  Backward, with dn_i = -(g_i . out_i) / n_i and dO = g / n prepared by
    // the caller: dQ's scores get + dn_i and its result + dn_i zc_c (dn, zc); dK's scores get + dn_i
    // (i: the dO row) and its result + rc_c (dn, rc).
    float *denom;     // fp32 [BH][N]
    float eps;
    const float *zc;  // fp32 [BH][n_chunks][D]: sum of k over the rows before chunk c
    const float *dn;  // fp32 [BH][N]
    const float *rc;  // fp32 [BH][n_chunks][D]: sum of dn_i q_i over the rows after chunk c
    // Forward, D = 128: where the state after the last chunk of every (b, h) goes, fp32 [BH][D][D]
    // ([q/k index][v index]), or null.  walk_bwd_rev_kernel: that buffer (xtotal) and forward's entry
    // states (xinit, the layout of `init`, not transposed; may be null with a single segment).
    float *total_out;
    const float *xinit, *xtotal;
    // D = 128, plain: the result (forward: o; walk_bwd_rev_kernel: dv) is added to what its place in
    // memory holds already -- the second of two walks whose results sum up (halves of a wide q / k)
    int32_t accumulate;
    // The wide walks (walk_fwd_wide_kernel, walk_bwd_rev_wide_kernel): q and k (dq and dk) have 129 .. 256
    // columns.  Columns 128 .. are the second half, of true width wqk2 (wqk = 128 is the first half's), with
    // entry and final states of its own in the layouts of init, total_out, xinit and xtotal.
    int32_t wqk2;
    const float *init2;
    float *total_out2;
    const float *xinit2, *xtotal2;
    // init_is_totals (every D = 128 walk; three segments or more): init (and init2) hold the segments' TOTALS as the
    // totals kernel wrote them, and a workgroup adds up those of the segments before its own (after it, walking in
    // reverse) as it starts, several loads in flight together -- no scan launch between the totals kernel and the
    // walk.  The forward walks (walk_fwd_kernel's plain D = 128 variant, walk_fwd_wide_kernel) then write the entry
    // state they formed to entry_out / entry_out2 (the layout of init; null: nowhere), for the backward walk.
    int32_t init_is_totals;
    float *entry_out, *entry_out2;
};

template <int D>
struct WalkCfg {
    static constexpr int C = walk_rows(D);  // rows per chunk
    static constexpr int RB = D * 2;        // bytes per tile row
    static constexpr int CR = D / 8;        // 16-byte chunks per row
    static constexpr int TILE = C * RB;     // bytes per operand tile
    static constexpr int KC = D / 16;       // 16-wide k chunks of a contraction over D
    static constexpr int DB = D / 32;       // 32-wide blocks of D
    static constexpr int RPI = 1024 / RB;   // rows covered by one wave-level 1 KiB load
    static constexpr int NI = TILE / 4096;  // such loads per wave and tile
    static constexpr int STATE = D * RB;    // the 16-bit state in LDS
    static constexpr int VEC = 3 * 1024;    // per set of tiles: zc, rc, dn of the chunk (fp32, 1 KiB each)
    static constexpr int NID = C / 64;      // wave-level 256-byte loads of a chunk's dn
    static constexpr int NBLK = DB * DB;    // 32 x 32 blocks of the state: block b belongs to wave b % 4
    static constexpr int NBW = (NBLK + 3) / 4;  // state blocks per wave
    // a wave owns one 32-row block of the chunk as the X rows of every product, and -- with fewer
    // than four such blocks -- one part of the output columns
    static constexpr int NRB = C / 32;      // row blocks per chunk
    static constexpr int NCH = 4 / NRB;     // column parts
    static constexpr int DBW = DB / NCH;    // 32-wide output blocks per wave
    static_assert(D == 32 || D == 64 || D == 128, "walk kernels are built for padded head dims 32, 64 and 128");
    static_assert(NRB * NCH == 4 && DBW * NCH == DB, "four waves tile the chunk's rows and output columns");
};

// The 32 x 32 blocks of the state that hold anything: NQ blocks of q/k indices (its rows), NV of v
// indices (its columns).  All D / 32 of each by default; the D = 128 kernels are also built for
// operands of at most 64 true columns on one side (NQ or NV = 2: the other blocks would hold the
// zeros the tiles are padded with, and the MFMAs on them are left out).
// State block i of wave `wave` is block wave + 4 i of the NQ x NV: (dbk, eb) = (block of q/k
// indices, block of v indices); the v block is the same for all blocks of a wave.
template <int D, int NQ = D / 32, int NV = D / 32>
struct WalkExt {
    static_assert(NQ >= 1 && NQ <= D / 32 && NV >= 1 && NV <= D / 32 && (4 % NV == 0 || NV % 4 == 0), "block counts");
    static constexpr int nq = NQ, nv = NV;
    static constexpr int SLOTS = (NQ * NV + 3) / 4;  // state blocks per wave
    static constexpr int KQ = 2 * NQ, KV = 2 * NV;   // 16-wide k chunks over the q/k side, the v side
    // (with a multiple of four blocks every slot of every wave holds one: known at compile time)
    __device__ static __forceinline__ bool valid(int wave, int i) { return (NQ * NV) % 4 == 0 || wave + 4 * i < NQ * NV; }
    __device__ static __forceinline__ int dbk(int wave, int i) { return (wave + 4 * i) / NV; }
    __device__ static __forceinline__ int eb(int wave) { return wave % NV; }
};

// Output blocks of a product whose result has NOB blocks that hold anything: with two column parts
// (D = 128) each part takes half of them -- PER blocks from block db0(wave).
template <int D, int NOB>
struct WalkOut {
    using W = WalkCfg<D>;
    static_assert(NOB % W::NCH == 0, "the column parts share the output blocks evenly");
    static constexpr int PER = NOB / W::NCH;
    __device__ static __forceinline__ int db0(int wave) { return W::NCH == 1 ? 0 : (wave / W::NRB) * PER; }
};

// ---- LDS tile access (tile: row-major [rows][D], chunk index XOR walk_swizzle(row))

// XOR applied to the 16-byte chunk index of tile row `row`.  Every tile is read both ways:
//   * along its rows (walk_row_frag): 16 lanes read the same chunk index of 16 consecutive rows,
//     which must land in the 16 different 16-byte slots of the 256 bytes that 64 banks span;
//   * down its columns (walk_col_frag*, transposing 8-byte reads): 32 lanes read 64 consecutive
//     bytes of each of 4 consecutive rows, which must land in 4 different 64-byte quarters.
// With 256-byte rows (D = 128) the row's low four bits go into the chunk index with its low two
// bits on top -- the bits that pick the 64-byte quarter -- and with 128-byte rows (D = 64, where
// the row's lowest bit already picks a half) bits 1 .. 3, bit 1 on top.  (Folding the bits in
// unpermuted serves the row reads just as well, but the 4 rows of a column read then meet in the
// same quarter: a 4-way bank conflict at D = 128, 2-way at D = 64.)
template <int CR>
__device__ __forceinline__ int walk_swizzle(int row) {
    if constexpr (CR == 4) {
        return (row >> 2) & 3;  // (64-byte rows: the 4 rows of a column read are the 4 quarters)
    } else if constexpr (CR == 8) {
        const int t = (row >> 1) & 7;
        return ((t & 1) << 2) | (t >> 1);
    } else {
        const int t = row & 15;
        return ((t & 3) << 2) | (t >> 2);
    }
}

// whole 128-row tile HBM -> LDS; rows >= N and chunks beyond the true width arrive as zeros
template <int D>
__device__ __forceinline__ void walk_load_tile(u32x4 rsrc, uint32_t lds_tile, int row0, int stride2, int width, int wave,
                                               int lane) {
    using W = WalkCfg<D>;
    const int r = wave * W::RPI + lane / W::CR;
    const int c = (lane % W::CR) ^ walk_swizzle<W::CR>(r);
    const uint32_t voff = (uint32_t)(r * stride2 + c * 16) + (c * 8 < width ? 0u : kOobOffset);
    const uint32_t base = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_tile + wave * 1024));
    u32x4 rs = {(uint32_t)__builtin_amdgcn_readfirstlane((int)rsrc[0]), (uint32_t)__builtin_amdgcn_readfirstlane((int)rsrc[1]),
                (uint32_t)__builtin_amdgcn_readfirstlane((int)rsrc[2]), (uint32_t)__builtin_amdgcn_readfirstlane((int)rsrc[3])};
    static_for<0, W::NI>([&](auto u) {
        constexpr int U = decltype(u)::value;
        const uint32_t so = (uint32_t)__builtin_amdgcn_readfirstlane((row0 + U * 4 * W::RPI) * stride2);
        dma_16B_per_lane<U * 4096>(rs, base, voff, so);
    });
}

// eight consecutive columns 16 kc + 8 g .. of one row: an MFMA operand with k along the row
template <typename T, int D>
__device__ __forceinline__ typename Mma<T>::V8 walk_row_frag(const unsigned char *tile, int row, int kc, int g) {
    using W = WalkCfg<D>;
    const int ch = (2 * kc + g) ^ walk_swizzle<W::CR>(row);
    return __builtin_bit_cast(typename Mma<T>::V8, *reinterpret_cast<const u32x4 *>(tile + row * W::RB + (ch << 4)));
}

__device__ __forceinline__ s16x4 walk_tr_read(const unsigned char *p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
}

// Column fragment with the output-column permutation of the product kernels: rows R0 + {4g .. 4g+3,
// 8+4g .. 8+4g+3} (the k order of a rounded S^T accumulator) of the 32 columns of block cb, taken
// so that MFMA row m = 8a + 4g' + b holds column 16g' + 4a + b -- a lane's 16 accumulator registers
// are then 16 consecutive output columns.  With `consecutive` the rows are R0 + 8g .. 8g+7 instead
// (the k order of a row fragment): the transposed read of the state.
template <typename T, int D>
__device__ __forceinline__ typename Mma<T>::V8 walk_col_frag_perm(const unsigned char *tile, int R0, int cb, int lane,
                                                                  bool consecutive) {
    using W = WalkCfg<D>;
    const int lam = lane & 15, g = lane >> 5, beta = (lane >> 4) & 1, zc = lam & 3;
    const int row_lo = R0 + (consecutive ? 8 * g : 4 * g) + (lam >> 2), row_hi = row_lo + (consecutive ? 4 : 8);
    const int ch = 4 * cb + 2 * (zc & 1) + beta, byte = 8 * (zc >> 1);
    const s16x4 lo = walk_tr_read(tile + row_lo * W::RB + ((ch ^ walk_swizzle<W::CR>(row_lo)) << 4) + byte);
    const s16x4 hi = walk_tr_read(tile + row_hi * W::RB + ((ch ^ walk_swizzle<W::CR>(row_hi)) << 4) + byte);
    return __builtin_bit_cast(typename Mma<T>::V8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// Column fragment, plain mapping (lane l32 <-> column 32 cb + l32), rows R0 + {4g.., 8+4g..}: both
// operands of the state update Y^T Z, whose contraction runs down the rows.
template <typename T, int D>
__device__ __forceinline__ typename Mma<T>::V8 walk_col_frag(const unsigned char *tile, int R0, int cb, int lane) {
    using W = WalkCfg<D>;
    const int lam = lane & 15, g = lane >> 5, beta = (lane >> 4) & 1;
    const int row_lo = R0 + 4 * g + (lam >> 2), row_hi = row_lo + 8;
    const int ch = 4 * cb + 2 * beta + ((lam & 3) >> 1), sub = 8 * (lam & 1);
    const s16x4 lo = walk_tr_read(tile + row_lo * W::RB + ((ch ^ walk_swizzle<W::CR>(row_lo)) << 4) + sub);
    const s16x4 hi = walk_tr_read(tile + row_hi * W::RB + ((ch ^ walk_swizzle<W::CR>(row_hi)) << 4) + sub);
    return __builtin_bit_cast(typename Mma<T>::V8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// MFMA row m of a state-product A operand holds output column e_lane(m) of its 32-column block
// (the permutation of walk_col_frag_perm)
__device__ __forceinline__ int walk_e_lane(int l32) { return 16 * ((l32 >> 2) & 1) + 4 * (l32 >> 3) + (l32 & 3); }

// ---- small fp32 vectors of a chunk HBM -> LDS (every wave issues them, to the same place)
template <int LDS_IMM>
__device__ __forceinline__ void dma_4B_per_lane(u32x4 rsrc, uint32_t lds_base, uint32_t voffset, uint32_t soffset) {
    asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset), "n"(LDS_IMM)
                 : "memory", "m0", "scc");
}
__device__ __forceinline__ u32x4 walk_uniform_rsrc(const void *base, uint32_t bytes) {
    const u32x4 r = make_rsrc(base, bytes);
    return u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)r[0]), (uint32_t)__builtin_amdgcn_readfirstlane((int)r[1]),
                 (uint32_t)__builtin_amdgcn_readfirstlane((int)r[2]), (uint32_t)__builtin_amdgcn_readfirstlane((int)r[3])};
}
// D floats (16-byte aligned) to lds_dst: one load, lanes beyond D / 4 write zeros (1 KiB is written)
template <int D>
__device__ __forceinline__ void walk_load_vec(const float *src, uint32_t lds_dst, int lane) {
    dma_16B_per_lane<0>(walk_uniform_rsrc(src, D * 4), (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst),
                        (uint32_t)lane * 16, 0);
}
// rows row0 .. row0 + C - 1 of a vector of N floats (zeros past the end) to lds_dst
template <int D>
__device__ __forceinline__ void walk_load_rows(const float *vec, int row0, int N, uint32_t lds_dst, int lane) {
    const u32x4 rs = walk_uniform_rsrc(vec + row0, (uint32_t)(N - row0) * 4);
    const uint32_t base = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
    static_for<0, WalkCfg<D>::NID>([&](auto u) {
        constexpr int U = decltype(u)::value;
        dma_4B_per_lane<U * 256>(rs, base, (uint32_t)lane * 4 + U * 256, 0);
    });
}

// acc[i][v] += scale * vec[32 (db0 + i) + 16 g + v] (vec: fp32 in LDS)
template <int D>
__device__ __forceinline__ void walk_add_vec(f32x16 (&acc)[WalkCfg<D>::DBW], float scale, const float *vec, int db0, int g) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));  // (declared again below, for the products)
#pragma unroll
    for (int i = 0; i < WalkCfg<D>::DBW; ++i)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const f32x4 z = *reinterpret_cast<const f32x4 *>(vec + 32 * (db0 + i) + 16 * g + 4 * a);
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[i][4 * a + b] += scale * z[b];
        }
}

// ---- one product of a chunk for this wave's 32 X rows (row block rb = wave % NRB) and its part of
// the output columns (blocks db0 .. db0 + DBW - 1, db0 = (wave / NRB) * DBW):
//   acc = [state: X_w . State]  +  mask(X_w Y^T) Z        (UPPER: keep row <= column, else row >= column)
// xt, yt, zt: LDS tiles; sfrag(db, kc): the state's A-operand fragment for output block db, k chunk kc.
// (With several column parts the waves of one row block each compute the same scores.)
// EX (the normaliser's terms): 1: ex = sum of this row's masked scores + x_row . exv (exv: D floats in
// LDS); 2: every score gets + ex (a value per X row, i.e. per lane) before the mask; 3: every
// score gets + exv[its Y row] (exv: one float per tile row, in LDS).
typedef float f32x4 __attribute__((ext_vector_type(4)));
struct WalkNoRows {
    __device__ __forceinline__ f32x4 operator()(int, int) const { return f32x4{0.f, 0.f, 0.f, 0.f}; }
};
// N operand fragments read from LDS and consumed in order, the read of fragment j + DEPTH issued
// before fragment j is used: use(j, fragment) for j = 0 .. N-1 with read(j + DEPTH) ahead of it.  The
// scheduling barriers keep the compiler from moving a read down to its use again (which it does when
// registers are scarce, and every MFMA then waits out the whole latency of its own LDS read).
template <int N, int DEPTH, typename V8, typename Read, typename Use>
__device__ __forceinline__ void walk_pipe(Read &&read, Use &&use) {
    V8 buf[N];
    static_for<0, (DEPTH < N ? DEPTH : N)>([&](auto j) { buf[decltype(j)::value] = read(j); });
    static_for<0, N>([&](auto j) {
        constexpr int J = decltype(j)::value;
        if constexpr (J + DEPTH < N) buf[J + DEPTH] = read(std::integral_constant<int, J + DEPTH>{});
        __builtin_amdgcn_sched_barrier(0);
        use(j, buf[J]);
    });
    __builtin_amdgcn_sched_barrier(0);
}

// KCL: 16-wide k chunks of the contraction X Y^T that hold anything; NOB: output blocks that do.
// KEEP: the product is added to what acc holds.
template <typename T, int D, bool UPPER, int EX = 0, int KCL = WalkCfg<D>::KC, int NOB = WalkCfg<D>::DB, bool KEEP = false,
          typename SFrag, typename YRows = WalkNoRows>
__device__ __forceinline__ void walk_product(const unsigned char *xt, const unsigned char *yt, const unsigned char *zt,
                                             int wave, int lane, bool has_state, SFrag &&sfrag,
                                             f32x16 (&acc)[WalkCfg<D>::DBW], float *ex = nullptr,
                                             const float *exv = nullptr, YRows &&yrows = WalkNoRows{}) {
    using W = WalkCfg<D>;
    using M = Mma<T>;
    using V8 = typename M::V8;
    constexpr int PER = WalkOut<D, NOB>::PER;
    const int l32 = lane & 31, g = lane >> 5;
    const int rb = W::NCH == 1 ? wave : wave % W::NRB, db0 = WalkOut<D, NOB>::db0(wave);
    V8 xf[KCL];
#pragma unroll
    for (int kc = 0; kc < KCL; ++kc) xf[kc] = walk_row_frag<T, D>(xt, 32 * rb + l32, kc, g);
    float rsum = 0.f;
    if constexpr (EX == 1) {
#pragma unroll
        for (int kc = 0; kc < KCL; ++kc)
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const f32x4 z = *reinterpret_cast<const f32x4 *>(exv + 16 * kc + 8 * g + 4 * a);
#pragma unroll
                for (int b = 0; b < 4; ++b) rsum += static_cast<float>(xf[kc][4 * a + b]) * z[b];
            }
    }
    if constexpr (!KEEP) {
#pragma unroll
        for (int i = 0; i < W::DBW; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
    }
    // One 32-row block s of Y and Z: scores, mask and rounding, second product.  ST: the state product's
    // MFMAs are issued in between -- PER / 2 of them after every score MFMA (they share its X fragment
    // and fill the gaps of the dependent chain), the rest after the last one, where the rounding of the
    // scores runs beneath them.  Operand fragments are read four ahead, in the order of their use.
    auto block = [&](int s, auto with_state) {
        constexpr bool ST = decltype(with_state)::value;
        constexpr int H = ST ? PER / 2 : 0, GA = 1 + H, GB = PER - H;
        constexpr int NA = KCL * GA, NB = ST ? GB * KCL : 0, NC = 2 * PER;
        constexpr int CONV = NB > 2 ? NA + 2 : NA + NB;  // the scores are finished in front of this operation
        f32x16 sc;
#pragma unroll
        for (int v = 0; v < 16; ++v) sc[v] = 0.f;
        V8 pf[2];
        walk_pipe<NA + NB + NC, 4, V8>(
            [&](auto j) {
                constexpr int J = decltype(j)::value;
                if constexpr (J < NA) {
                    if constexpr (J % GA == 0)
                        return walk_row_frag<T, D>(yt, 32 * s + l32, J / GA, g);
                    else
                        return sfrag(db0 + J % GA - 1, J / GA);
                } else if constexpr (J < NA + NB) {
                    return sfrag(db0 + H + (J - NA) % GB, (J - NA) / GB);
                } else {
                    return walk_col_frag_perm<T, D>(zt, 32 * s + 16 * ((J - NA - NB) / PER), db0 + (J - NA - NB) % PER, lane,
                                                    false);
                }
            },
            [&](auto j, V8 f) {
                constexpr int J = decltype(j)::value;
                if constexpr (J == CONV) {  // normaliser's terms, mask, rounding
                    if constexpr (EX == 2) {
#pragma unroll
                        for (int v = 0; v < 16; ++v) sc[v] += *ex;
                    }
                    if constexpr (EX == 3) {
#pragma unroll
                        for (int a = 0; a < 4; ++a) {
                            const f32x4 y = yrows(s, a);
#pragma unroll
                            for (int b = 0; b < 4; ++b) sc[4 * a + b] += y[b];
                        }
                    }
                    if (s == rb) {  // the 32 x 32 block on the diagonal: lane = X row l32, register v = Y row jl
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int jl = 8 * (v / 4) + 4 * g + (v % 4);
                            const bool keep = UPPER ? l32 <= jl : l32 >= jl;
                            sc[v] = keep ? sc[v] : 0.f;
                        }
                    }
                    if constexpr (EX == 1) {
#pragma unroll
                        for (int v = 0; v < 16; ++v) rsum += sc[v];
                    }
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int e = 0; e < 8; ++e) pf[t][e] = static_cast<T>(sc[8 * t + e]);
                }
                if constexpr (J < NA) {
                    if constexpr (J % GA == 0)
                        sc = M::mma(f, xf[J / GA], sc);
                    else
                        acc[J % GA - 1] = M::mma(f, xf[J / GA], acc[J % GA - 1]);
                } else if constexpr (J < NA + NB) {
                    acc[H + (J - NA) % GB] = M::mma(f, xf[(J - NA) / GB], acc[H + (J - NA) % GB]);
                } else {
                    acc[(J - NA - NB) % PER] = M::mma(f, pf[(J - NA - NB) / PER], acc[(J - NA - NB) % PER]);
                }
            });
    };
    const int s_lo = UPPER ? rb : 0, s_hi = UPPER ? W::NRB - 1 : rb;
    if constexpr (D == 128) {
        if (has_state)
            block(s_lo, std::true_type{});
        else
            block(s_lo, std::false_type{});
#pragma unroll 1
        for (int s = s_lo + 1; s <= s_hi; ++s) block(s, std::false_type{});
    } else {
        // (two workgroups per CU cover each other's gaps, and the fused backward has no registers to
        // spare for the longer pipeline: the state product on its own, k chunk outer, output block inner)
        if (has_state) {
            walk_pipe<PER * KCL, 4, V8>([&](auto j) { return sfrag(db0 + decltype(j)::value % PER, decltype(j)::value / PER); },
                                        [&](auto j, V8 f) {
                                            constexpr int I = decltype(j)::value % PER, KC_ = decltype(j)::value / PER;
                                            acc[I] = M::mma(f, xf[KC_], acc[I]);
                                        });
        }
#pragma unroll 1
        for (int s = s_lo; s <= s_hi; ++s) block(s, std::false_type{});
    }
    if constexpr (EX == 1) *ex = rsum + __shfl_xor(rsum, 32, 64);  // the two lanes of a row hold half the columns each
}

// Every element of the landed tile replaced by phi(element), in place, and the mapped rows written
// to `out` (rows >= N and chunks beyond the true width arrived as zeros and stay zeros).  The
// caller synchronises before the tile is read.
template <typename T, int D>
__device__ __forceinline__ void walk_map_tile(unsigned char *tile, int fmap, int row0, int N, int width, T *out,
                                              int64_t out_stride, int tid) {
    using W = WalkCfg<D>;
    feature_dispatch(fmap, [&](auto map) {
#pragma unroll
        for (int v = 0; v < W::C * W::CR / 256; ++v) {
            const int u = tid + 256 * v, r = u / W::CR, pos = u % W::CR, c = pos ^ walk_swizzle<W::CR>(r);
            if (row0 + r < N && c * 8 < width) {
                u32x4 *ptr = reinterpret_cast<u32x4 *>(tile + r * W::RB + (pos << 4));
                const u32x4 m = feature_map8_c<T, decltype(map)::value>(*ptr);
                *ptr = m;
                *reinterpret_cast<u32x4 *>(out + (int64_t)(row0 + r) * out_stride + c * 8) = m;
            }
        }
    });
}

// acc[i][v] = Out[row][32 (db0 + i) + 16 g + v] rounded to the storage type: pk[i][hq] = columns
// 32 (db0 + i) + 16 g + 8 hq .. + 7.  With a feature map, `ytile` is the LDS tile holding
// y = phi(x) for the same rows (tile row `trow`) and Out is multiplied by the slope phi'(x),
// computed from y, first.
template <typename T, int D, int PER = WalkCfg<D>::DBW>
__device__ __forceinline__ void walk_pack(const f32x16 (&acc)[WalkCfg<D>::DBW], int g, int db0,
                                          u32x4 (&pk)[WalkCfg<D>::DBW][2], int fmap = 0,
                                          const unsigned char *ytile = nullptr, int trow = 0) {
    using W = WalkCfg<D>;
    using V8 = typename Mma<T>::V8;
    float sl[PER][2][8];  // the slopes (one branch on the map around all of them)
    if (fmap) {
        feature_dispatch(fmap, [&](auto map) {
#pragma unroll
            for (int i = 0; i < PER; ++i)
#pragma unroll
                for (int hq = 0; hq < 2; ++hq) {
                    const int ch = (4 * (db0 + i) + 2 * g + hq) ^ walk_swizzle<W::CR>(trow);
                    const V8 y = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4 *>(ytile + trow * W::RB + (ch << 4)));
#pragma unroll
                    for (int e = 0; e < 8; ++e) sl[i][hq][e] = feature_slope_c<decltype(map)::value>(static_cast<float>(y[e]));
                }
        });
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
#pragma unroll
        for (int hq = 0; hq < 2; ++hq) {
            V8 o8;
#pragma unroll
            for (int e = 0; e < 8; ++e) o8[e] = static_cast<T>(fmap ? acc[i][8 * hq + e] * sl[i][hq][e] : acc[i][8 * hq + e]);
            pk[i][hq] = __builtin_bit_cast(u32x4, o8);
        }
    }
}

// two 16-byte stores per block; rows >= N and columns beyond the true width fall outside the
// buffer resource and are dropped
template <int D, int PER = WalkCfg<D>::DBW>
__device__ __forceinline__ void walk_store_packed(__amdgpu_buffer_rsrc_t rs, int stride2, int width, int row, int g,
                                                  int db0, const u32x4 (&pk)[WalkCfg<D>::DBW][2]) {
#pragma unroll
    for (int i = 0; i < PER; ++i)
#pragma unroll
        for (int hq = 0; hq < 2; ++hq) {
            const int col = 32 * (db0 + i) + 16 * g + 8 * hq;
            const uint32_t off = (uint32_t)(row * stride2 + col * 2) + (col < width ? 0u : kOobOffset);
            __builtin_amdgcn_raw_buffer_store_b128(pk[i][hq], rs, off, 0, 0);
        }
}

// (PER: the blocks of acc that are this wave's -- the others belong to another wave or hold nothing)
template <typename T, int D, int PER = WalkCfg<D>::DBW>
__device__ __forceinline__ void walk_store(__amdgpu_buffer_rsrc_t rs, int stride2, int width, int row, int g, int db0,
                                           const f32x16 (&acc)[WalkCfg<D>::DBW], int fmap = 0,
                                           const unsigned char *ytile = nullptr, int trow = 0) {
    u32x4 pk[WalkCfg<D>::DBW][2];
    walk_pack<T, D, PER>(acc, g, db0, pk, fmap, ytile, trow);
    walk_store_packed<D, PER>(rs, stride2, width, row, g, db0, pk);
}

// What a result's place in memory holds before the walk adds to it: this lane's 16-byte pieces of the
// row it will store (the pieces of walk_store_packed).  Ordinary loads, requested once a chunk's tiles
// have been awaited and used at the end of the chunk: the wait the compiler puts in front of the use
// also covers the tile loads of the next chunk, issued before the request -- by then they have had
// the whole chunk's time to land.
template <typename T, int D, int PER>
struct WalkPrev {
    u32x4 val[PER][2];
    __device__ __forceinline__ void request(__amdgpu_buffer_rsrc_t rs, int stride2, int width, int row, int g, int db0) {
#pragma unroll
        for (int i = 0; i < PER; ++i)
#pragma unroll
            for (int hq = 0; hq < 2; ++hq) {
                const int col = 32 * (db0 + i) + 16 * g + 8 * hq;
                const uint32_t off = (uint32_t)(row * stride2 + col * 2) + (col < width ? 0u : kOobOffset);
                val[i][hq] = __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0);
            }
    }
    __device__ __forceinline__ void add_to(f32x16 (&acc)[WalkCfg<D>::DBW]) const {
        typedef T v8 __attribute__((ext_vector_type(8)));
#pragma unroll
        for (int i = 0; i < PER; ++i)
#pragma unroll
            for (int hq = 0; hq < 2; ++hq) {
                const v8 y = __builtin_bit_cast(v8, val[i][hq]);
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[i][8 * hq + e] += static_cast<float>(y[e]);
            }
    }
};

// state += Y^T Z over the rows of the tiles, this wave's 32 x 32 blocks (block i: Y columns of block
// dbk(i), Z columns of block eb): st[i][v] = State[32 dbk(i) + 8(v/4) + 4g + v%4][32 eb + l32]
// (NEG: state -= Y^T Z -- the sign bits of the Z fragments are flipped.  ACC: the state lives in
// accumulation registers, see Mma::mma_acc; the wait states an MFMA's result needs before anything
// but another MFMA reads it are spent at the end, since the compiler does not count them for a
// statement it cannot look into.)
template <typename T, int D, typename B = WalkExt<D>, bool NEG = false, bool ACC = false>
__device__ __forceinline__ void walk_update(const unsigned char *yt, const unsigned char *zt, int wave, int lane,
                                            f32x16 (&st)[WalkCfg<D>::NBW]) {
    using W = WalkCfg<D>;
    using M = Mma<T>;
    using V8 = typename M::V8;
    if (!B::valid(wave, 0)) return;
    // per 16 rows: the Z fragment, then the Y fragment of every block -- one group of reads ahead of the MFMAs
    constexpr int G = 1 + B::SLOTS, KS = W::C / 16;
    V8 zf = {};
    walk_pipe<KS * G, G, V8>(
        [&](auto j) {
            constexpr int ks = decltype(j)::value / G, r = decltype(j)::value % G;
            if constexpr (r == 0) {
                V8 z = walk_col_frag<T, D>(zt, 16 * ks, B::eb(wave), lane);
                if constexpr (NEG) {
                    u32x4 raw = __builtin_bit_cast(u32x4, z);
#pragma unroll
                    for (int e = 0; e < 4; ++e) raw[e] ^= 0x80008000u;
                    z = __builtin_bit_cast(V8, raw);
                }
                return z;
            } else {
                // (a slot without a block -- only in the last one, with fewer than four blocks in all -- reads block 0)
                return walk_col_frag<T, D>(yt, 16 * ks, B::valid(wave, r - 1) ? B::dbk(wave, r - 1) : 0, lane);
            }
        },
        [&](auto j, V8 f) {
            constexpr int r = decltype(j)::value % G;
            if constexpr (r == 0) {
                zf = f;
            } else if (B::valid(wave, r - 1)) {
                if constexpr (ACC)
                    M::mma_acc(f, zf, st[r - 1]);
                else
                    st[r - 1] = M::mma(f, zf, st[r - 1]);
            }
        });
    if constexpr (ACC) {
        static_assert(!ACC || B::SLOTS == 4 || B::SLOTS == 2, "written for two or four blocks per wave");
        if constexpr (B::SLOTS == 4)
            asm volatile("s_nop 15\n\ts_nop 7" : "+a"(st[0]), "+a"(st[1]), "+a"(st[2]), "+a"(st[3]));
        else
            asm volatile("s_nop 15\n\ts_nop 7" : "+a"(st[0]), "+a"(st[1]));
    }
}

// the state rounded to 16 bit into LDS as T[v index][q/k index] (row = 32 eb + l32, four consecutive
// columns per register group), in the tile layout
template <typename T, int D, typename B = WalkExt<D>>
__device__ __forceinline__ void walk_state_to_lds(unsigned char *tl, int wave, int lane,
                                                  const f32x16 (&st)[WalkCfg<D>::NBW]) {
    using W = WalkCfg<D>;
    typedef T t4 __attribute__((ext_vector_type(4)));
    const int l32 = lane & 31, g = lane >> 5, row = 32 * B::eb(wave) + l32;
#pragma unroll
    for (int i = 0; i < B::SLOTS; ++i) {
        if (!B::valid(wave, i)) continue;
        const int dbk = B::dbk(wave, i);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            t4 w;
#pragma unroll
            for (int b = 0; b < 4; ++b) w[b] = static_cast<T>(st[i][4 * a + b]);
            *reinterpret_cast<t4 *>(tl + row * W::RB + (((4 * dbk + a) ^ walk_swizzle<W::CR>(row)) << 4) + 8 * g) = w;
        }
    }
}

struct WalkSlice {
    int bh, seg, c_lo, c_hi;  // chunks c_lo .. c_hi - 1
    bool valid;
};

// workgroup -> ((b, h), segment): heads of one XCD in sequence, as in the other kernels
__device__ __forceinline__ WalkSlice walk_slice(const WalkParams &p) {
    const int wg = blockIdx.x, xcd = wg & 7, slot = wg >> 3;
    const int hl = slot / p.n_seg, seg = slot - hl * p.n_seg;
    WalkSlice s;
    s.bh = hl * 8 + xcd, s.seg = seg;
    s.c_lo = seg * p.seg_chunks;
    s.c_hi = s.c_lo + p.seg_chunks < p.n_chunks ? s.c_lo + p.seg_chunks : p.n_chunks;
    s.valid = s.bh < p.BH && s.c_lo < p.n_chunks;
    return s;
}

// this wave's blocks of an fp32 state [D][D] in memory, assigned to st or (ADD) added to it;
// `transposed`: the buffer holds the transposed matrix ([v index][q/k index])
template <int D, typename B, bool ADD>
__device__ __forceinline__ void walk_read_state(const float *init, bool transposed, int wave, int lane,
                                                f32x16 (&st)[WalkCfg<D>::NBW]) {
    const int l32 = lane & 31, g = lane >> 5;
    // st[i][v] = State[r = 32 dbk(i) + 8 (v/4) + 4g + v%4][c = 32 eb + l32]: element r D + c of the
    // buffer, or c D + r when it holds the transposed matrix (then four consecutive floats per v/4)
    const int c = 32 * B::eb(wave) + l32;
    if (transposed) {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int i = 0; i < B::SLOTS; ++i)
            if (B::valid(wave, i)) {
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const f32x4 t = *reinterpret_cast<const f32x4 *>(init + c * D + 32 * B::dbk(wave, i) + 8 * a + 4 * g);
#pragma unroll
                    for (int b = 0; b < 4; ++b) st[i][4 * a + b] = ADD ? st[i][4 * a + b] + t[b] : t[b];
                }
            }
    } else {
#pragma unroll
        for (int i = 0; i < B::SLOTS; ++i)
            if (B::valid(wave, i)) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float t = init[(32 * B::dbk(wave, i) + 8 * (v / 4) + 4 * g + (v % 4)) * D + c];
                    st[i][v] = ADD ? st[i][v] + t : t;
                }
            }
    }
}

// ... zeros for a null pointer; with `init2` the state is the sum of the two buffers
template <int D, typename B = WalkExt<D>>
__device__ __forceinline__ void walk_load_state(const float *init, bool transposed, int wave, int lane,
                                                f32x16 (&st)[WalkCfg<D>::NBW], const float *init2 = nullptr) {
    using W = WalkCfg<D>;
#pragma unroll
    for (int i = 0; i < W::NBW; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) st[i][v] = 0.f;
    if (!init) return;
    walk_read_state<D, B, false>(init, transposed, wave, lane, st);
    if (init2) walk_read_state<D, B, true>(init2, transposed, wave, lane, st);
}

// Entry states in memory, fp32 [D][D] per segment, [bh][seg], in one of three forms that host and
// kernels tell apart by the number of segments alone:
//   * two segments per (b, h): the first segment in walking order starts from zero and the other one
//     from the one total the totals kernel forms; its two workgroups of a (b, h) add up half of that
//     segment each, and the two slots hold their partial sums;
//   * three to walk_sum_on_load_max(D) segments: the slots hold the segments' TOTALS as the totals kernel
//     wrote them, and a walk adds up the totals of the segments before it (after it, walking in reverse)
//     as it starts -- a few states of D x D read from L2 per workgroup instead of a scan kernel between
//     the totals kernel and the walk, whose launch costs more than it computes on plans this small
//     (B H = 16, N = 1024, D = 64, forward + backward: 40.7 -> 32.8 us, bound by its six -> four launches);
//   * more segments: the slots hold the entry states themselves (walk_scan_kernel).
// Padded head dims up to 64 only.  At D = 128 a workgroup has its CU to itself and nothing hides the
// latency of those reads at its start: with four segments the forward walk gained 10 us and the reverse
// walk, which starts from two such sums, lost 60 (B 4, H 16, N 4096, D_qk 256 as two halves: 0.333 -> 0.384 ms).
__host__ __device__ constexpr int walk_sum_on_load_max(int D) { return D <= 64 ? 8 : 0; }
__host__ __device__ constexpr bool walk_entries_are_totals(int D, int n_seg) {
    return n_seg >= 3 && n_seg <= walk_sum_on_load_max(D);
}

// this wave's blocks of the sum of the states buf[f_lo .. f_hi - 1] (zeros for an empty range), added in
// ascending order, the loads of up to four states (two of four blocks per wave) in flight together (one state at a time is a chain of
// dependent loads: a memory latency per state at the start of every workgroup)
template <int D, typename B>
__device__ __forceinline__ void walk_sum_states(const float *buf, int f_lo, int f_hi, bool transposed, int wave, int lane,
                                                f32x16 (&st)[WalkCfg<D>::NBW]) {
    using W = WalkCfg<D>;
    constexpr int GROUP = B::SLOTS > 2 ? 2 : 4;  // (GROUP x SLOTS x 16 registers beside the sum)
#pragma unroll
    for (int i = 0; i < W::NBW; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) st[i][v] = 0.f;
#pragma unroll 1
    for (int f0 = f_lo; f0 < f_hi; f0 += GROUP) {
        f32x16 t[GROUP][W::NBW];
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            const int f = f0 + u < f_hi ? f0 + u : f_hi - 1;  // (past the range: the last state once more, not added)
            walk_read_state<D, B, false>(buf + (int64_t)f * (D * D), transposed, wave, lane, t[u]);
        }
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            const float keep = f0 + u < f_hi ? 1.f : 0.f;
#pragma unroll
            for (int i = 0; i < B::SLOTS; ++i)
                if (B::valid(wave, i)) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) st[i][v] += keep * t[u][i][v];
                }
        }
    }
}

// st_a, st_b = this wave's blocks of the sums of the states a[f_lo .. f_hi - 1], b[f_lo .. f_hi - 1], the loads of
// up to three states of each in flight together (a chain of dependent loads costs a memory latency per state)
template <int D, typename B>
__device__ __forceinline__ void walk_sum_two(const float *a, const float *b, int f_lo, int f_hi, int wave, int lane,
                                             f32x16 (&st_a)[WalkCfg<D>::NBW], f32x16 (&st_b)[WalkCfg<D>::NBW]) {
    using W = WalkCfg<D>;
    constexpr int E = D * D, GROUP = 3;
    static_assert(B::SLOTS <= 2, "2 x GROUP x SLOTS x 16 registers beside the two sums: for states of two blocks per wave");
#pragma unroll
    for (int i = 0; i < W::NBW; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) st_a[i][v] = 0.f, st_b[i][v] = 0.f;
#pragma unroll 1
    for (int f0 = f_lo; f0 < f_hi; f0 += GROUP) {
        f32x16 ta[GROUP][W::NBW], tb[GROUP][W::NBW];
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            // (past the range: the last state once more, not added)
            const int f = f0 + u < f_hi ? f0 + u : f_hi - 1;
            walk_read_state<D, B, false>(a + (int64_t)f * E, false, wave, lane, ta[u]);
            walk_read_state<D, B, false>(b + (int64_t)f * E, false, wave, lane, tb[u]);
        }
#pragma unroll
        for (int u = 0; u < GROUP; ++u) {
            const float keep = f0 + u < f_hi ? 1.f : 0.f;
#pragma unroll
            for (int i = 0; i < B::SLOTS; ++i)
                if (B::valid(wave, i)) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) st_a[i][v] += keep * ta[u][i][v], st_b[i][v] += keep * tb[u][i][v];
                }
        }
    }
}

// this wave's blocks of the entry state of segment sl.seg (zeros without a buffer) of a walk in
// ascending (`reverse` false) or descending order of the chunks; `buf`: the entry states of one operand
template <int D, typename B = WalkExt<D>>
__device__ __forceinline__ void walk_load_init_from(const float *buf, const WalkParams &p, const WalkSlice &sl, int wave,
                                                    int lane, f32x16 (&st)[WalkCfg<D>::NBW], bool reverse) {
    const float *init = nullptr, *init2 = nullptr;
    if (buf) {
        if (p.n_seg == 2) {
            if (sl.seg != (reverse ? 1 : 0)) init = buf + (int64_t)sl.bh * 2 * (D * D), init2 = init + D * D;
        } else if (walk_entries_are_totals(D, p.n_seg) || p.init_is_totals) {
            walk_sum_states<D, B>(buf + (int64_t)sl.bh * p.n_seg * (D * D), reverse ? sl.seg + 1 : 0,
                                  reverse ? p.n_seg : sl.seg, p.init_transposed != 0, wave, lane, st);
            return;
        } else {
            init = buf + ((int64_t)sl.bh * p.n_seg + sl.seg) * (D * D);
        }
    }
    walk_load_state<D, B>(init, p.init_transposed != 0, wave, lane, st, init2);
}
template <int D, typename B = WalkExt<D>>
__device__ __forceinline__ void walk_load_init(const WalkParams &p, const WalkSlice &sl, int wave, int lane,
                                               f32x16 (&st)[WalkCfg<D>::NBW], bool reverse) {
    walk_load_init_from<D, B>(p.init, p, sl, wave, lane, st, reverse);
}

// the forward state at the end of segment sl.seg from what forward handed over: the entry state of
// the next segment (xinit, in the forms above) or, for the last one, the final state (xtotal)
template <int D, typename B = WalkExt<D>>
__device__ __forceinline__ void walk_load_end_state_from(const float *xinit, const float *xtotal, const WalkParams &p,
                                                         const WalkSlice &sl, int wave, int lane,
                                                         f32x16 (&xs)[WalkCfg<D>::NBW]) {
    const float *x = xtotal + (int64_t)sl.bh * (D * D), *x2 = nullptr;
    if (sl.c_hi < p.n_chunks) {
        if (p.n_seg == 2) {
            x = xinit + (int64_t)sl.bh * 2 * (D * D), x2 = x + D * D;
        } else if (walk_entries_are_totals(D, p.n_seg)) {
            walk_sum_states<D, B>(xinit + (int64_t)sl.bh * p.n_seg * (D * D), 0, sl.seg + 1, false, wave, lane, xs);
            return;
        } else {
            x = xinit + ((int64_t)sl.bh * p.n_seg + sl.seg + 1) * (D * D);
        }
    }
    walk_load_state<D, B>(x, false, wave, lane, xs, x2);
}
template <int D, typename B = WalkExt<D>>
__device__ __forceinline__ void walk_load_end_state(const WalkParams &p, const WalkSlice &sl, int wave, int lane,
                                                    f32x16 (&xs)[WalkCfg<D>::NBW]) {
    walk_load_end_state_from<D, B>(p.xinit, p.xtotal, p, sl, wave, lane, xs);
}

// this wave's blocks of a state to an fp32 buffer [D][D] ([q/k index][v index]); blocks outside B stay unwritten
template <int D, typename B>
__device__ __forceinline__ void walk_write_state(float *out, int wave, int lane, const f32x16 (&st)[WalkCfg<D>::NBW]) {
    const int l32 = lane & 31, g = lane >> 5;
#pragma unroll
    for (int i = 0; i < B::SLOTS; ++i)
        if (B::valid(wave, i)) {
#pragma unroll
            for (int v = 0; v < 16; ++v)
                out[(32 * B::dbk(wave, i) + 8 * (v / 4) + 4 * g + (v % 4)) * D + 32 * B::eb(wave) + l32] = st[i][v];
        }
}

// ---- one product with its running state, chunks ascending:
//   O_c = lower(Q_c K_c^T) V_c + Q_c S, then S += K_c^T V_c
// (forward as named; dQ of the split backward with q <- dO, k <- V, v <- K, o <- dQ and the entry
// states read transposed)
// DOUBLE: one workgroup per CU with two sets of tiles -- the loads of the next chunk are in flight
// while this one is multiplied.  (Holding a chunk's results back and storing them after the next
// chunk's tiles have been awaited, so that the wait for the tiles never includes fresh stores,
// measured 20 % slower: the stores then compete with the loads in flight instead of filling the
// gap after them.)
// NORM: the instantiations that take the normaliser's terms: 1 forward (WalkParams::denom), 2 dQ (dn).
// FM: the instantiations that know of feature maps (WalkParams::fmap, slope_y); the others ignore both.
// NQ, NV: blocks of the state [q/k index][v index] that hold anything (WalkExt).
// ACCUM: the result is added to what o holds already (WalkParams::accumulate, WalkPrev).
template <typename T, int D, bool DOUBLE, int NORM, bool FM, int NQ = D / 32, int NV = D / 32, bool ACCUM = false>
__global__ __launch_bounds__(256, DOUBLE ? 1 : 2) void walk_fwd_kernel(const WalkParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    using W = WalkCfg<D>;
    using V8 = typename Mma<T>::V8;
    using B = WalkExt<D, NQ, NV>;
    using OB = WalkOut<D, NV>;  // the result is as wide as v
    static_assert(NORM == 0 || (NQ == W::DB && NV == W::DB), "the normaliser's variants are built for full widths");
    static_assert(!ACCUM || (DOUBLE && NORM == 0 && !FM), "adding to the result: the plain D = 128 walk only");
    constexpr int SETS = DOUBLE ? 2 : 1;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    unsigned char *tl = smem + SETS * 3 * W::TILE;
    unsigned char *xv = tl + W::STATE;  // per set: zc, (unused), dn of the chunk
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rb = W::NCH == 1 ? wave : wave % W::NRB, db0 = OB::db0(wave);
    const WalkSlice sl = walk_slice(p);
    if (!sl.valid) return;
    const int fmap = FM ? p.fmap : 0;
    const void *slope_y = FM ? p.slope_y : nullptr;
    const int b = sl.bh / p.H, h = sl.bh - b * p.H, N = p.N;
    const T *Q = static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h;
    const T *K = static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h;
    const T *V = static_cast<const T *>(p.v) + b * p.vs_b + h * p.vs_h;
    T *O = static_cast<T *>(p.o) + b * p.os_b + h * p.os_h;
    const int qs2 = (int)p.qs_n * 2, ks2 = (int)p.ks_n * 2, vs2 = (int)p.vs_n * 2, os2 = (int)p.os_n * 2;
    const u32x4 rq = make_rsrc(Q, (uint32_t)((N - 1) * qs2 + p.wqk * 2));
    const u32x4 rk = make_rsrc(K, (uint32_t)((N - 1) * ks2 + p.wqk * 2));
    const u32x4 rv = make_rsrc(V, (uint32_t)((N - 1) * vs2 + p.wv * 2));
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(O, 0, (N - 1) * os2 + p.wv * 2, 0x00020000);

    f32x16 st[W::NBW];
    walk_load_init<D, B>(p, sl, wave, lane, st, false);
    if constexpr (DOUBLE && NORM == 0 && !FM) {  // (the entry state this walk formed from the segments' totals, for backward)
        if (p.init_is_totals && p.entry_out && sl.seg > 0)
            walk_write_state<D, B>(p.entry_out + ((int64_t)sl.bh * p.n_seg + sl.seg) * (D * D), wave, lane, st);
    }
    walk_state_to_lds<T, D, B>(tl, wave, lane, st);

    auto load_chunk = [&](int c, int buf) {
        const uint32_t base = lds0 + buf * 3 * W::TILE;
        walk_load_tile<D>(rq, base, c * W::C, qs2, p.wqk, wave, lane);
        walk_load_tile<D>(rk, base + W::TILE, c * W::C, ks2, p.wqk, wave, lane);
        walk_load_tile<D>(rv, base + 2 * W::TILE, c * W::C, vs2, p.wv, wave, lane);
        const uint32_t xbase = lds0 + SETS * 3 * W::TILE + W::STATE + buf * W::VEC;
        if constexpr (NORM) {
            walk_load_vec<D>(p.zc + ((int64_t)sl.bh * p.n_chunks + c) * D, xbase, lane);
            if constexpr (NORM == 2) walk_load_rows<D>(p.dn + (int64_t)sl.bh * N, c * W::C, N, xbase + 2048, lane);
        }
    };
    constexpr int n_extra = NORM == 0 ? 0 : NORM == 1 ? 1 : 1 + W::NID;  // loads per chunk and wave beyond the tiles
    // ACCUM: the result is added to what o holds (in fp32, before the one rounding)
    WalkPrev<T, D, OB::PER> prev;
    if constexpr (DOUBLE) load_chunk(sl.c_lo, 0);
#pragma unroll 1
    for (int c = sl.c_lo; c < sl.c_hi; ++c) {
        const int row0 = c * W::C, buf = DOUBLE ? (c - sl.c_lo) & 1 : 0;
        unsigned char *tq = smem + buf * 3 * W::TILE, *tk = tq + W::TILE, *tv = tq + 2 * W::TILE;
        const int row = row0 + 32 * rb + l32;
        // dQ walk with a feature map: this lane's values of phi(xq) under its accumulator registers,
        // requested before the tiles so that they have arrived with them
        V8 ys[W::DBW][2];
        if (slope_y) {
            const T *yrow = static_cast<const T *>(slope_y) + b * p.sy_b + h * p.sy_h + (int64_t)(row < N ? row : 0) * p.sy_n;
#pragma unroll
            for (int i = 0; i < W::DBW; ++i)
#pragma unroll
                for (int hq = 0; hq < 2; ++hq) {
                    const int col = 32 * (db0 + i) + 16 * g + 8 * hq;
                    u32x4 raw = {0u, 0u, 0u, 0u};
                    if (col < p.wv) raw = *reinterpret_cast<const u32x4 *>(yrow + col);
                    ys[i][hq] = __builtin_bit_cast(V8, raw);
                }
        }
        if constexpr (DOUBLE) {
            const bool more = c + 1 < sl.c_hi;
            if (more) load_chunk(c + 1, buf ^ 1);  // (every wave has left the barrier that ended the reads of that set)
            // this wave's loads of chunk c have landed when at most the loads issued after them are
            // outstanding (the stores of the previous chunk were issued before those)
            if (more)
                wait_vm<3 * W::NI + n_extra>();
            else
                wait_vm<0>();
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's part of the state is in LDS
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (fmap && p.qmap_out) {
                walk_map_tile<T, D>(tq, fmap, row0, N, p.wqk, static_cast<T *>(p.qmap_out) + b * p.qo_b + h * p.qo_h,
                                    p.qo_n, tid);
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the rewritten tile is in LDS
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
        } else {
            load_chunk(c, 0);
            wait_vm<0>();
            __syncthreads();  // the tiles have landed; the state written by the previous iteration is visible
            if (fmap && p.qmap_out) {
                walk_map_tile<T, D>(tq, fmap, row0, N, p.wqk, static_cast<T *>(p.qmap_out) + b * p.qo_b + h * p.qo_h,
                                    p.qo_n, tid);
                __syncthreads();
            }
        }
        if constexpr (ACCUM) prev.request(ro, os2, p.wv, row, g, db0);
        f32x16 acc[W::DBW];
        const float *vz = reinterpret_cast<const float *>(xv + buf * W::VEC);
        const float *vd = reinterpret_cast<const float *>(xv + buf * W::VEC + 2048);
        auto sfrag = [&](int db, int kc) -> V8 { return walk_row_frag<T, D>(tl, 32 * db + walk_e_lane(l32), kc, g); };
        if constexpr (NORM == 1) {  // forward with the normaliser: n = masked row sum + q . zc + eps
            float tot;
            walk_product<T, D, false, 1, B::KQ, NV>(tq, tk, tv, wave, lane, c > 0, sfrag, acc, &tot, vz);
            const float n = tot + p.eps, inv = 1.0f / n;
#pragma unroll
            for (int i = 0; i < W::DBW; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][v] *= inv;
            if (db0 == 0 && g == 0 && row < N) p.denom[(int64_t)sl.bh * N + row] = n;
        } else if constexpr (NORM == 2) {  // dQ with the normaliser's term: scores + dn_i, result + dn_i zc
            float ax = vd[32 * rb + l32];
            walk_product<T, D, false, 2, B::KQ, NV>(tq, tk, tv, wave, lane, c > 0, sfrag, acc, &ax);
            walk_add_vec<D>(acc, ax, vz, db0, g);
        } else {
            walk_product<T, D, false, 0, B::KQ, NV>(tq, tk, tv, wave, lane, c > 0, sfrag, acc);
        }
        if (slope_y) {
            feature_dispatch(fmap, [&](auto map) {
#pragma unroll
                for (int i = 0; i < W::DBW; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        acc[i][v] *= feature_slope_c<decltype(map)::value>(static_cast<float>(ys[i][v / 8][v % 8]));
            });
        }
        if constexpr (ACCUM) prev.add_to(acc);
        walk_store<T, D, OB::PER>(ro, os2, p.wv, row, g, db0, acc);
        if (!DOUBLE && p.saved) {  // the state at the entry of this chunk, [q/k index][v index], for backward's dQ
            T *sv = static_cast<T *>(p.saved) + ((int64_t)sl.bh * p.n_chunks + c) * (D * D);
#pragma unroll
            for (int i = 0; i < B::SLOTS; ++i)
                if (B::valid(wave, i)) {
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        sv[(32 * B::dbk(wave, i) + 8 * (v / 4) + 4 * g + (v % 4)) * D + 32 * B::eb(wave) + l32] =
                            static_cast<T>(st[i][v]);
                }
        }
        walk_update<T, D, B>(tk, tv, wave, lane, st);
        if constexpr (DOUBLE) {
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0xc07f);  // this wave's LDS reads of the tiles and of the state are done
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else {
            __syncthreads();  // every wave is done with the tiles and with the old state
        }
        walk_state_to_lds<T, D, B>(tl, wave, lane, st);
    }
    if (p.total_out && sl.c_hi == p.n_chunks) {  // the state after the last chunk, for the backward walks
        float *out = p.total_out + (int64_t)sl.bh * (D * D);
#pragma unroll
        for (int i = 0; i < B::SLOTS; ++i)
            if (B::valid(wave, i)) {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    out[(32 * B::dbk(wave, i) + 8 * (v / 4) + 4 * g + (v % 4)) * D + 32 * B::eb(wave) + l32] = st[i][v];
            }
        // (built for a narrow q / k side: walk_bwd_rev_kernel has no such variant and reads every block)
        if constexpr (NQ < W::DB) {
            for (int e = tid; e < D * D; e += 256)
                if (e / D >= 32 * NQ || e % D >= 32 * NV) out[e] = 0.f;
        }
    }
#else
    (void)p;
#endif
}

// ---- forward for q and k of 129 .. 256 columns (v of at most 128), one walk over both 128-column halves:
//   O_c = sum over the halves h of lower(Q_h,c K_h,c^T) V_c + Q_h,c S_h,   then S_h += K_h,c^T V_c
// Each half is the D = 128 product of walk_fwd_kernel with a state of its own; the chunk's result stays in
// its fp32 accumulators from the first half to the second and is rounded and stored once, and V is loaded
// once per chunk -- where two walks of walk_fwd_kernel, the second adding to the first one's result, load V
// twice, write O twice and read it back once.
// LDS: a set of (Q_h, K_h) tiles per half -- while half h of a chunk is multiplied, the loads of the next
// half-chunk go to the other set -- two V tiles (chunk parity), and ONE 16-bit state: a half's state is
// needed in LDS only for that half's product, so at the end of a half-chunk the other half's state (in
// registers throughout, updated one half-chunk earlier) is rounded into the buffer.
// NV: the state's v blocks that hold anything (2: v of at most 64 columns).
template <typename T, int NV>
__global__ __launch_bounds__(256, 1) void walk_fwd_wide_kernel(const WalkParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int D = 128;
    using W = WalkCfg<D>;
    using V8 = typename Mma<T>::V8;
    using B = WalkExt<D, D / 32, NV>;
    using OB = WalkOut<D, NV>;  // the result is as wide as v
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    unsigned char *tl = smem + 6 * W::TILE;
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rb = wave % W::NRB, db0 = OB::db0(wave);
    const WalkSlice sl = walk_slice(p);
    if (!sl.valid) return;
    const int b = sl.bh / p.H, h = sl.bh - b * p.H, N = p.N;
    const T *Q = static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h;
    const T *K = static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h;
    const T *V = static_cast<const T *>(p.v) + b * p.vs_b + h * p.vs_h;
    T *O = static_cast<T *>(p.o) + b * p.os_b + h * p.os_h;
    const int qs2 = (int)p.qs_n * 2, ks2 = (int)p.ks_n * 2, vs2 = (int)p.vs_n * 2, os2 = (int)p.os_n * 2;
    const u32x4 rq0 = make_rsrc(Q, (uint32_t)((N - 1) * qs2 + p.wqk * 2));
    const u32x4 rk0 = make_rsrc(K, (uint32_t)((N - 1) * ks2 + p.wqk * 2));
    const u32x4 rq1 = make_rsrc(Q + D, (uint32_t)((N - 1) * qs2 + p.wqk2 * 2));
    const u32x4 rk1 = make_rsrc(K + D, (uint32_t)((N - 1) * ks2 + p.wqk2 * 2));
    const u32x4 rv = make_rsrc(V, (uint32_t)((N - 1) * vs2 + p.wv * 2));
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(O, 0, (N - 1) * os2 + p.wv * 2, 0x00020000);

    f32x16 st0[W::NBW], st1[W::NBW];
    if (p.init_is_totals) {
        const int64_t at = (int64_t)sl.bh * p.n_seg * (D * D);
        if constexpr (NV == 2) {  // (both halves' loads in flight together; with four blocks per wave and state, one half's)
            walk_sum_two<D, B>(p.init + at, p.init2 + at, 0, sl.seg, wave, lane, st0, st1);
        } else {
            walk_sum_states<D, B>(p.init + at, 0, sl.seg, false, wave, lane, st0);
            walk_sum_states<D, B>(p.init2 + at, 0, sl.seg, false, wave, lane, st1);
        }
        if (p.entry_out && sl.seg > 0) {  // (the first segment's entry state, zero, is read by nobody)
            walk_write_state<D, B>(p.entry_out + at + (int64_t)sl.seg * (D * D), wave, lane, st0);
            walk_write_state<D, B>(p.entry_out2 + at + (int64_t)sl.seg * (D * D), wave, lane, st1);
        }
    } else {
        walk_load_init_from<D, B>(p.init, p, sl, wave, lane, st0, false);
        walk_load_init_from<D, B>(p.init2, p, sl, wave, lane, st1, false);
    }
    walk_state_to_lds<T, D, B>(tl, wave, lane, st0);

    auto load_half = [&](int c, auto half) {  // Q_h, K_h of chunk c to set h
        constexpr int HF = decltype(half)::value;
        const uint32_t base = lds0 + HF * 2 * W::TILE;
        walk_load_tile<D>(HF ? rq1 : rq0, base, c * W::C, qs2, HF ? p.wqk2 : p.wqk, wave, lane);
        walk_load_tile<D>(HF ? rk1 : rk0, base + W::TILE, c * W::C, ks2, HF ? p.wqk2 : p.wqk, wave, lane);
    };
    auto v_slot = [&](int c) { return 4 + ((c - sl.c_lo) & 1); };
    auto load_v = [&](int c) { walk_load_tile<D>(rv, lds0 + v_slot(c) * W::TILE, c * W::C, vs2, p.wv, wave, lane); };
    auto sync = [&]() {  // this wave's LDS accesses are done; then every wave's
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    auto sfrag = [&](int db, int kc) -> V8 { return walk_row_frag<T, D>(tl, 32 * db + walk_e_lane(l32), kc, g); };
    load_half(sl.c_lo, std::integral_constant<int, 0>{});
    load_v(sl.c_lo);
#pragma unroll 1
    for (int c = sl.c_lo; c < sl.c_hi; ++c) {
        unsigned char *tq0 = smem, *tk0 = smem + W::TILE, *tq1 = smem + 2 * W::TILE, *tk1 = smem + 3 * W::TILE;
        unsigned char *tv = smem + v_slot(c) * W::TILE;
        const int row = c * W::C + 32 * rb + l32;
        f32x16 acc[W::DBW];
        // first half.  (Every wave has left the barrier that ended the reads of the set loaded next, one
        // half-chunk ago.)  This wave's loads of the half-chunk have landed when at most the loads issued
        // after them are outstanding; the stores of the chunk before were issued before those.
        load_half(c, std::integral_constant<int, 1>{});
        wait_vm<2 * W::NI>();
        sync();  // the tiles have landed, S_0 is in LDS
        walk_product<T, D, false, 0, B::KQ, NV>(tq0, tk0, tv, wave, lane, c > 0, sfrag, acc);
        walk_update<T, D, B>(tk0, tv, wave, lane, st0);
        sync();  // every wave has read S_0 and this half's tiles
        walk_state_to_lds<T, D, B>(tl, wave, lane, st1);
        // second half
        const bool more = c + 1 < sl.c_hi;
        if (more) {
            load_half(c + 1, std::integral_constant<int, 0>{});
            load_v(c + 1);  // (to the slot of the chunk before this one)
            wait_vm<3 * W::NI>();
        } else {
            wait_vm<0>();
        }
        sync();  // the tiles have landed, S_1 is in LDS
        walk_product<T, D, false, 0, B::KQ, NV, true>(tq1, tk1, tv, wave, lane, c > 0, sfrag, acc);
        walk_store<T, D, OB::PER>(ro, os2, p.wv, row, g, db0, acc);
        walk_update<T, D, B>(tk1, tv, wave, lane, st1);
        sync();  // every wave has read S_1, this half's tiles and V
        walk_state_to_lds<T, D, B>(tl, wave, lane, st0);
    }
    if (p.total_out && sl.c_hi == p.n_chunks) {  // the states after the last chunk, for the backward walk
        walk_write_state<D, B>(p.total_out + (int64_t)sl.bh * (D * D), wave, lane, st0);
        walk_write_state<D, B>(p.total_out2 + (int64_t)sl.bh * (D * D), wave, lane, st1);
        // (NV = 2: the v blocks beyond stay unwritten -- walk_bwd_rev_wide_kernel, the reader, is built for the same extent)
    }
#else
    (void)p;
#endif
}

// ---- backward: dQ, dV, dK of a chunk from one set of tiles; R += Q_c^T dO_c, chunks descending.
// dQ's state, the sum of K^T V over the chunks before:
//   NORM (the normaliser's terms): the 16-bit state forward saved at the entry of every chunk
//   (WalkParams::saved), fragments straight from memory;
//   otherwise obtained backwards as in walk_bwd_rev_kernel: X starts as the forward state at the
//   segment's end (xinit / xtotal) and every chunk's K^T V is subtracted when the walk reaches it;
//   X has a 16-bit copy of its own in LDS beside R's.  Forward then saves no per-chunk states.
template <typename T, int D, bool NORM>
__global__ __launch_bounds__(256, 2) void walk_bwd_kernel(const WalkParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    using W = WalkCfg<D>;
    using V8 = typename Mma<T>::V8;
    static_assert(W::NCH == 1, "the fused backward keeps dQ's state fragments of all output blocks in registers");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    unsigned char *tq = smem, *tk = smem + W::TILE, *tv = smem + 2 * W::TILE, *tg = smem + 3 * W::TILE,
                  *tl = smem + 4 * W::TILE;
    unsigned char *tx = tl + W::STATE;  // (!NORM) X's copy; (NORM) the chunk's vectors
    const float *vz = reinterpret_cast<const float *>(tl + W::STATE), *vr = vz + 256, *vd = vz + 512;
    const uint32_t xbase = lds0 + 4 * W::TILE + W::STATE;
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const WalkSlice sl = walk_slice(p);
    if (!sl.valid) return;
    const int b = sl.bh / p.H, h = sl.bh - b * p.H, N = p.N;
    const T *Q = static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h;
    const T *K = static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h;
    const T *V = static_cast<const T *>(p.v) + b * p.vs_b + h * p.vs_h;
    const T *G = static_cast<const T *>(p.go) + b * p.gs_b + h * p.gs_h;
    T *DQ = static_cast<T *>(p.dq) + b * p.dqs_b + h * p.dqs_h;
    T *DK = static_cast<T *>(p.dk) + b * p.dks_b + h * p.dks_h;
    T *DV = static_cast<T *>(p.dv) + b * p.dvs_b + h * p.dvs_h;
    const int qs2 = (int)p.qs_n * 2, ks2 = (int)p.ks_n * 2, vs2 = (int)p.vs_n * 2, gs2 = (int)p.gs_n * 2;
    const int dqs2 = (int)p.dqs_n * 2, dks2 = (int)p.dks_n * 2, dvs2 = (int)p.dvs_n * 2;
    const u32x4 rq = make_rsrc(Q, (uint32_t)((N - 1) * qs2 + p.wqk * 2));
    const u32x4 rk = make_rsrc(K, (uint32_t)((N - 1) * ks2 + p.wqk * 2));
    const u32x4 rv = make_rsrc(V, (uint32_t)((N - 1) * vs2 + p.wv * 2));
    const u32x4 rg = make_rsrc(G, (uint32_t)((N - 1) * gs2 + p.wv * 2));
    const __amdgpu_buffer_rsrc_t rdq = __builtin_amdgcn_make_buffer_rsrc(DQ, 0, (N - 1) * dqs2 + p.wqk * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rdk = __builtin_amdgcn_make_buffer_rsrc(DK, 0, (N - 1) * dks2 + p.wqk * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rdv = __builtin_amdgcn_make_buffer_rsrc(DV, 0, (N - 1) * dvs2 + p.wv * 2, 0x00020000);

    f32x16 st[W::NBW];  // R[q/k index][v index]
    walk_load_init<D>(p, sl, wave, lane, st, true);
    walk_state_to_lds<T, D>(tl, wave, lane, st);
    f32x16 xs[W::NBW];  // X[q/k index][v index]
    if constexpr (!NORM)
        walk_load_end_state<D>(p, sl, wave, lane, xs);

#pragma unroll 1
    for (int c = sl.c_hi - 1; c >= sl.c_lo; --c) {
        const int row0 = c * W::C;
        walk_load_tile<D>(rq, lds0, row0, qs2, p.wqk, wave, lane);
        walk_load_tile<D>(rk, lds0 + W::TILE, row0, ks2, p.wqk, wave, lane);
        walk_load_tile<D>(rv, lds0 + 2 * W::TILE, row0, vs2, p.wv, wave, lane);
        walk_load_tile<D>(rg, lds0 + 3 * W::TILE, row0, gs2, p.wv, wave, lane);
        if constexpr (NORM) {  // the normaliser's terms: zc, rc of this chunk and its rows of dn
            walk_load_vec<D>(p.zc + ((int64_t)sl.bh * p.n_chunks + c) * D, xbase, lane);
            walk_load_vec<D>(p.rc + ((int64_t)sl.bh * p.n_chunks + c) * D, xbase + 1024, lane);
            walk_load_rows<D>(p.dn + (int64_t)sl.bh * N, row0, N, xbase + 2048, lane);
        }
        // NORM: dQ's state, S_c[q/k index][v index] as saved by forward: A-operand fragments straight from
        // memory (row = output column of dQ, eight consecutive v indices)
        V8 sfq[NORM ? W::DB : 1][NORM ? W::KC : 1];
        if constexpr (NORM) {
            const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
                static_cast<T *>(p.saved) + ((int64_t)sl.bh * p.n_chunks + c) * (D * D), 0, D * D * 2, 0x00020000);
            if (c > 0) {
#pragma unroll
                for (int db = 0; db < W::DB; ++db)
#pragma unroll
                    for (int kc = 0; kc < W::KC; ++kc)
                        sfq[db][kc] = __builtin_bit_cast(V8, __builtin_amdgcn_raw_buffer_load_b128(
                                                                 rs, (uint32_t)(((32 * db + walk_e_lane(l32)) * D + 16 * kc + 8 * g) * 2), 0, 0));
            }
        }
        wait_vm<0>();
        __syncthreads();
        const int row = row0 + 32 * wave + l32;
        const bool later = c + 1 < p.n_chunks;  // chunks after this one exist: R is not identically zero
        f32x16 acc[W::DBW];
        if constexpr (NORM) {
            // dQ = lower(dO V^T) K + dO S_c^T  (normaliser: scores + dn_i, result + dn_i zc)
            float ax = vd[32 * wave + l32];
            walk_product<T, D, false, 2>(tg, tv, tk, wave, lane, c > 0, [&](int db, int kc) -> V8 { return sfq[db][kc]; },
                                         acc, &ax);
            walk_add_vec<D>(acc, ax, vz, 0, g);
            walk_store<T, D>(rdq, dqs2, p.wqk, row, g, 0, acc, p.fmap, tq, 32 * wave + l32);
        } else {
            walk_update<T, D, WalkExt<D>, true>(tk, tv, wave, lane, xs);  // X: now the sum over the chunks before this one
            walk_state_to_lds<T, D>(tx, wave, lane, xs);
        }
        // dV = upper(K Q^T) dO + K R: A operand R^T[v index][q/k index] = the LDS copy as it is
        walk_product<T, D, true>(tk, tq, tg, wave, lane, later, [&](int db, int kc) -> V8 {
            return walk_row_frag<T, D>(tl, 32 * db + walk_e_lane(l32), kc, g);
        }, acc);
        walk_store<T, D>(rdv, dvs2, p.wv, row, g, 0, acc);
        // dK = upper(V dO^T) Q + V R^T: A operand R[q/k index][v index] = the LDS copy read transposed
        // (normaliser: scores + dn_i with i the dO row, result + rc)
        if constexpr (NORM) {
            walk_product<T, D, true, 3>(tv, tg, tq, wave, lane, later, [&](int db, int kc) -> V8 {
                return walk_col_frag_perm<T, D>(tl, 16 * kc, db, lane, true);
            }, acc, nullptr, nullptr, [&](int s, int a) -> f32x4 {
                return *reinterpret_cast<const f32x4 *>(vd + 32 * s + 8 * a + 4 * g);
            });
            walk_add_vec<D>(acc, 1.0f, vr, 0, g);
        } else {
            walk_product<T, D, true>(tv, tg, tq, wave, lane, later, [&](int db, int kc) -> V8 {
                return walk_col_frag_perm<T, D>(tl, 16 * kc, db, lane, true);
            }, acc);
        }
        walk_store<T, D>(rdk, dks2, p.wqk, row, g, 0, acc, p.fmap, tk, 32 * wave + l32);
        if constexpr (!NORM) {
            __syncthreads();  // every wave's part of X is in LDS
            // dQ = lower(dO V^T) K + dO X^T: A operand X[q/k index][v index], its LDS copy read transposed
            walk_product<T, D, false>(tg, tv, tk, wave, lane, c > 0, [&](int db, int kc) -> V8 {
                return walk_col_frag_perm<T, D>(tx, 16 * kc, db, lane, true);
            }, acc);
            walk_store<T, D>(rdq, dqs2, p.wqk, row, g, 0, acc, p.fmap, tq, 32 * wave + l32);
        }
        walk_update<T, D>(tq, tg, wave, lane, st);
        __syncthreads();
        walk_state_to_lds<T, D>(tl, wave, lane, st);
    }
#else
    (void)p;
#endif
}

// ---- backward without saved per-chunk states, dV and dK: chunks descending, R += Q_c^T dO_c.  One
// workgroup per CU with two sets of tiles: the loads of the next chunk are in flight while this
// one is multiplied.  (dQ is a walk_fwd_kernel launch over dO, V, K.)
// NORM: dK with the normaliser's terms (scores + dn_i, i the dO row; result + rc).  Tiles and state
// fill the LDS at D = 128, so the chunk's dn and this wave's columns of rc travel in registers: a
// lane loads one value of each, a chunk ahead, and the values are handed round within the wave
// (ds_bpermute: 64 per chunk, about 30 clocks each -- 28 us of a 207 us launch at B H = 128,
// N = 4096) when the chunk's turn comes.
template <typename T, int D, bool NORM, int NQ = D / 32, int NV = D / 32>
__global__ __launch_bounds__(256, 1) void walk_dkdv_kernel(const WalkParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    using W = WalkCfg<D>;
    using V8 = typename Mma<T>::V8;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    unsigned char *tl = smem + 8 * W::TILE;
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    using B = WalkExt<D, NQ, NV>;   // R [q/k index][v index]
    using OV = WalkOut<D, NV>;      // dV is as wide as v,
    using OQ = WalkOut<D, NQ>;      // dK as q and k
    static_assert(!NORM || (NQ == W::DB && NV == W::DB), "the normaliser's variant is built for full widths");
    const int rb = W::NCH == 1 ? wave : wave % W::NRB, db0 = OQ::db0(wave);  // (db0: dK's, and rc's columns)
    const WalkSlice sl = walk_slice(p);
    if (!sl.valid) return;
    const int b = sl.bh / p.H, h = sl.bh - b * p.H, N = p.N;
    const T *Q = static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h;
    const T *K = static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h;
    const T *V = static_cast<const T *>(p.v) + b * p.vs_b + h * p.vs_h;
    const T *G = static_cast<const T *>(p.go) + b * p.gs_b + h * p.gs_h;
    T *DK = static_cast<T *>(p.dk) + b * p.dks_b + h * p.dks_h;
    T *DV = static_cast<T *>(p.dv) + b * p.dvs_b + h * p.dvs_h;
    const int qs2 = (int)p.qs_n * 2, ks2 = (int)p.ks_n * 2, vs2 = (int)p.vs_n * 2, gs2 = (int)p.gs_n * 2;
    const int dks2 = (int)p.dks_n * 2, dvs2 = (int)p.dvs_n * 2;
    const u32x4 rq = make_rsrc(Q, (uint32_t)((N - 1) * qs2 + p.wqk * 2));
    const u32x4 rk = make_rsrc(K, (uint32_t)((N - 1) * ks2 + p.wqk * 2));
    const u32x4 rv = make_rsrc(V, (uint32_t)((N - 1) * vs2 + p.wv * 2));
    const u32x4 rg = make_rsrc(G, (uint32_t)((N - 1) * gs2 + p.wv * 2));
    const __amdgpu_buffer_rsrc_t rdk = __builtin_amdgcn_make_buffer_rsrc(DK, 0, (N - 1) * dks2 + p.wqk * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rdv = __builtin_amdgcn_make_buffer_rsrc(DV, 0, (N - 1) * dvs2 + p.wv * 2, 0x00020000);

    f32x16 st[W::NBW];  // R[q/k index][v index]
    walk_load_init<D, B>(p, sl, wave, lane, st, true);
    walk_state_to_lds<T, D, B>(tl, wave, lane, st);

    auto load_chunk = [&](int c, int buf) {
        const uint32_t base = lds0 + buf * 4 * W::TILE;
        const int row0 = c * W::C;
        walk_load_tile<D>(rq, base, row0, qs2, p.wqk, wave, lane);
        walk_load_tile<D>(rk, base + W::TILE, row0, ks2, p.wqk, wave, lane);
        walk_load_tile<D>(rv, base + 2 * W::TILE, row0, vs2, p.wv, wave, lane);
        walk_load_tile<D>(rg, base + 3 * W::TILE, row0, gs2, p.wv, wave, lane);
    };
    static_assert(!NORM || W::C == 64, "one dn value per lane covers a chunk of 64 rows");
    // Ordinary loads, requested a chunk ahead (once the tiles of the chunk before have been awaited) and
    // read at the top of their chunk, BEFORE the next tile loads go out: the wait the compiler puts
    // in front of the first use is one for every outstanding load and store (it cannot count past
    // stores), and at that point nothing is in flight that the walk would not wait for anyway but the
    // previous chunk's stores, issued two products earlier.
    float nxt_dn = 0.f, nxt_rc = 0.f;
    // (rows past the end read as zero; without the normaliser the two descriptors are never used)
    const __amdgpu_buffer_rsrc_t rs_dn =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(NORM ? p.dn + (int64_t)sl.bh * N : nullptr), 0, NORM ? N * 4 : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_rc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(NORM ? p.rc + (int64_t)sl.bh * p.n_chunks * D : nullptr), 0, NORM ? p.n_chunks * D * 4 : 0, 0x00020000);
    auto load_vecs = [&](int c) {  // lane l: dn of row l of chunk c, rc of column 32 db0 + l
        if constexpr (NORM) {
            nxt_dn = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_dn, (c * W::C + lane) * 4, 0, 0));
            nxt_rc = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_rc, (c * D + 32 * db0 + lane) * 4, 0, 0));
        }
    };
    load_chunk(sl.c_hi - 1, 0);
    load_vecs(sl.c_hi - 1);
#pragma unroll 1
    for (int c = sl.c_hi - 1; c >= sl.c_lo; --c) {
        const int buf = (sl.c_hi - 1 - c) & 1;
        unsigned char *tq = smem + buf * 4 * W::TILE, *tk = tq + W::TILE, *tv = tq + 2 * W::TILE, *tg = tq + 3 * W::TILE;
        const bool more = c > sl.c_lo;
        // this chunk's vectors, from the lanes that loaded them: dnv[a][b] = dn of tile row 8 a + 4 g + b,
        // rcv[i][v] = rc of column 32 (db0 + i) + 16 g + v
        f32x4 dnv[8];
        f32x16 rcv[W::DBW];
        if constexpr (NORM) {
#pragma unroll
            for (int a8 = 0; a8 < 8; ++a8)
#pragma unroll
                for (int b4 = 0; b4 < 4; ++b4) dnv[a8][b4] = __shfl(nxt_dn, 8 * a8 + 4 * g + b4, 64);
#pragma unroll
            for (int i = 0; i < W::DBW; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) rcv[i][v] = __shfl(nxt_rc, 32 * i + 16 * g + v, 64);
            asm volatile("" ::"v"(dnv[7]), "v"(rcv[W::DBW - 1]) : "memory");  // (handed round before the tile loads below)
        }
        if (more) load_chunk(c - 1, buf ^ 1);  // (every wave has left the barrier that ended the reads of that set)
        // this wave's loads of chunk c have landed when at most the loads issued after them are
        // outstanding (the stores of the previous chunk were issued before those)
        if (more)
            wait_vm<4 * W::NI>();
        else
            wait_vm<0>();
        if constexpr (NORM) {
            if (more) load_vecs(c - 1);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's part of the state is in LDS
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const int row = c * W::C + 32 * rb + l32;
        const bool later = c + 1 < p.n_chunks;  // chunks after this one exist: R is not identically zero
        f32x16 acc[W::DBW];
        // dV = upper(K Q^T) dO + K R: A operand R^T[v index][q/k index] = the LDS copy as it is
        walk_product<T, D, true, 0, B::KQ, NV>(tk, tq, tg, wave, lane, later, [&](int db, int kc) -> V8 {
            return walk_row_frag<T, D>(tl, 32 * db + walk_e_lane(l32), kc, g);
        }, acc);
        walk_store<T, D, OV::PER>(rdv, dvs2, p.wv, row, g, OV::db0(wave), acc);
        // dK = upper(V dO^T) Q + V R^T: A operand R[q/k index][v index] = the LDS copy read transposed
        if constexpr (NORM) {
            walk_product<T, D, true, 3>(tv, tg, tq, wave, lane, later, [&](int db, int kc) -> V8 {
                return walk_col_frag_perm<T, D>(tl, 16 * kc, db, lane, true);
            }, acc, nullptr, nullptr, [&](int s, int a4) -> f32x4 { return s == 0 ? dnv[a4] : dnv[4 + a4]; });
#pragma unroll
            for (int i = 0; i < W::DBW; ++i) acc[i] += rcv[i];
        } else {
            walk_product<T, D, true, 0, B::KV, NQ>(tv, tg, tq, wave, lane, later, [&](int db, int kc) -> V8 {
                return walk_col_frag_perm<T, D>(tl, 16 * kc, db, lane, true);
            }, acc);
        }
        walk_store<T, D, OQ::PER>(rdk, dks2, p.wqk, row, g, db0, acc, p.fmap, tk, 32 * rb + l32);
        walk_update<T, D, B>(tq, tg, wave, lane, st);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xc07f);  // this wave's LDS reads of the tiles and of the state are done
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        walk_state_to_lds<T, D, B>(tl, wave, lane, st);
    }
#else
    (void)p;
#endif
}

// ---- backward at D = 128 in one reverse walk: dV, dK and dQ of a chunk from one set of tiles.
//   R = sum of Q^T dO over the chunks after this one, as in walk_dkdv_kernel;
//   X = sum of K^T V over the chunks before it, obtained backwards: X starts as the forward state at
//   the end of the segment (the next segment's entry state, or the state after the last chunk) and
//   every chunk's K^T V is subtracted when the walk reaches it.  (In fp32: the difference carries
//   the rounding of the sums it is taken from, about 1e-7 of the largest state -- far below the
//   16-bit rounding the state gets before it multiplies dO.)
// The one 16-bit state in LDS holds R for dV and dK, then X for dQ.  q, k, v, dO are read once and
// nothing but the results is written, where the walk for dQ followed by walk_dkdv_kernel reads
// dO, v, k twice.
template <typename T, int D, int NQ = D / 32, int NV = D / 32, bool ACCUM = false, bool FM = false>
__global__ __launch_bounds__(256, 1) void walk_bwd_rev_kernel(const WalkParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    using W = WalkCfg<D>;
    using V8 = typename Mma<T>::V8;
    using B = WalkExt<D, NQ, NV>;   // R, X [q/k index][v index]
    using OV = WalkOut<D, NV>;      // dV is as wide as v,
    using OQ = WalkOut<D, NQ>;      // dK and dQ as q and k
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    unsigned char *tl = smem + 8 * W::TILE;
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rb = W::NCH == 1 ? wave : wave % W::NRB;
    const WalkSlice sl = walk_slice(p);
    if (!sl.valid) return;
    // FM: q and k hold y = phi(x); dQ and dK leave multiplied by the slope of phi, computed from the tiles
    const int fmap = FM ? p.fmap : 0;
    const int b = sl.bh / p.H, h = sl.bh - b * p.H, N = p.N;
    const T *Q = static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h;
    const T *K = static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h;
    const T *V = static_cast<const T *>(p.v) + b * p.vs_b + h * p.vs_h;
    const T *G = static_cast<const T *>(p.go) + b * p.gs_b + h * p.gs_h;
    T *DQ = static_cast<T *>(p.dq) + b * p.dqs_b + h * p.dqs_h;
    T *DK = static_cast<T *>(p.dk) + b * p.dks_b + h * p.dks_h;
    T *DV = static_cast<T *>(p.dv) + b * p.dvs_b + h * p.dvs_h;
    const int qs2 = (int)p.qs_n * 2, ks2 = (int)p.ks_n * 2, vs2 = (int)p.vs_n * 2, gs2 = (int)p.gs_n * 2;
    const int dqs2 = (int)p.dqs_n * 2, dks2 = (int)p.dks_n * 2, dvs2 = (int)p.dvs_n * 2;
    const u32x4 rq = make_rsrc(Q, (uint32_t)((N - 1) * qs2 + p.wqk * 2));
    const u32x4 rk = make_rsrc(K, (uint32_t)((N - 1) * ks2 + p.wqk * 2));
    const u32x4 rv = make_rsrc(V, (uint32_t)((N - 1) * vs2 + p.wv * 2));
    const u32x4 rg = make_rsrc(G, (uint32_t)((N - 1) * gs2 + p.wv * 2));
    const __amdgpu_buffer_rsrc_t rdq = __builtin_amdgcn_make_buffer_rsrc(DQ, 0, (N - 1) * dqs2 + p.wqk * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rdk = __builtin_amdgcn_make_buffer_rsrc(DK, 0, (N - 1) * dks2 + p.wqk * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rdv = __builtin_amdgcn_make_buffer_rsrc(DV, 0, (N - 1) * dvs2 + p.wv * 2, 0x00020000);

    f32x16 st[W::NBW];  // R [q/k index][v index]
    f32x16 xs[W::NBW];  // X [q/k index][v index]
    walk_load_init<D, B>(p, sl, wave, lane, st, true);
    walk_load_end_state<D, B>(p, sl, wave, lane, xs);
    walk_state_to_lds<T, D, B>(tl, wave, lane, st);

    auto load_chunk = [&](int c, int buf) {
        const uint32_t base = lds0 + buf * 4 * W::TILE;
        const int row0 = c * W::C;
        walk_load_tile<D>(rq, base, row0, qs2, p.wqk, wave, lane);
        walk_load_tile<D>(rk, base + W::TILE, row0, ks2, p.wqk, wave, lane);
        walk_load_tile<D>(rv, base + 2 * W::TILE, row0, vs2, p.wv, wave, lane);
        walk_load_tile<D>(rg, base + 3 * W::TILE, row0, gs2, p.wv, wave, lane);
    };
    auto sync = [&]() {  // this wave's LDS accesses are done; then every wave's
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    // ACCUM: dV is added to what dv holds (in fp32, before the one rounding)
    WalkPrev<T, D, OV::PER> prev;
    load_chunk(sl.c_hi - 1, 0);
#pragma unroll 1
    for (int c = sl.c_hi - 1; c >= sl.c_lo; --c) {
        const int buf = (sl.c_hi - 1 - c) & 1;
        unsigned char *tq = smem + buf * 4 * W::TILE, *tk = tq + W::TILE, *tv = tq + 2 * W::TILE, *tg = tq + 3 * W::TILE;
        const bool more = c > sl.c_lo;
        if (more) load_chunk(c - 1, buf ^ 1);  // (every wave has left the barrier that ended the reads of that set)
        // this wave's loads of chunk c have landed when at most the loads issued after them are
        // outstanding (the stores of the previous chunk were issued before those)
        if (more)
            wait_vm<4 * W::NI>();
        else
            wait_vm<0>();
        sync();  // the tiles have landed, R is in LDS
        const int row = c * W::C + 32 * rb + l32;
        const bool later = c + 1 < p.n_chunks;  // chunks after this one exist: R is not identically zero
        if constexpr (ACCUM) prev.request(rdv, dvs2, p.wv, row, g, OV::db0(wave));
        walk_update<T, D, B, true, true>(tk, tv, wave, lane, xs);  // X: now the sum over the chunks before this one
        f32x16 acc[W::DBW];
        // dV = upper(K Q^T) dO + K R: A operand R^T[v index][q/k index] = the LDS copy as it is
        walk_product<T, D, true, 0, B::KQ, NV>(tk, tq, tg, wave, lane, later, [&](int db, int kc) -> V8 {
            return walk_row_frag<T, D>(tl, 32 * db + walk_e_lane(l32), kc, g);
        }, acc);
        f32x16 held[W::DBW];  // ACCUM: dV waits for the end of the chunk (see WalkPrev)
        if constexpr (ACCUM) {
#pragma unroll
            for (int i = 0; i < OV::PER; ++i) held[i] = acc[i];
        } else {
            walk_store<T, D, OV::PER>(rdv, dvs2, p.wv, row, g, OV::db0(wave), acc);
        }
        // dK = upper(V dO^T) Q + V R^T: A operand R[q/k index][v index] = the LDS copy read transposed
        walk_product<T, D, true, 0, B::KV, NQ>(tv, tg, tq, wave, lane, later, [&](int db, int kc) -> V8 {
            return walk_col_frag_perm<T, D>(tl, 16 * kc, db, lane, true);
        }, acc);
        walk_store<T, D, OQ::PER>(rdk, dks2, p.wqk, row, g, OQ::db0(wave), acc, fmap, tk, 32 * rb + l32);
        // R += Q^T dO touches registers and tiles only, so it can sit on either side of the barriers: the waves of
        // the last row block, with one score block in dV and dK against two, take it here, the others after dQ,
        // where they have one score block against two
        // (full widths only: with a narrow v side the balance is the other way round, measured)
        constexpr bool kSplitUpdate = W::NRB == 2 && NQ == W::DB && NV == W::DB;
        if (kSplitUpdate && rb == 1) walk_update<T, D, B, false, true>(tq, tg, wave, lane, st);
        sync();  // every wave has read R
        // (X stays in its accumulation registers up to here: without this the copies that the rounding
        // below reads are made right after the update and occupy 64 registers through both products)
        if constexpr (B::SLOTS == 4)
            asm volatile("" : "+a"(xs[0]), "+a"(xs[1]), "+a"(xs[2]), "+a"(xs[3]));
        else
            asm volatile("" : "+a"(xs[0]), "+a"(xs[1]));
        walk_state_to_lds<T, D, B>(tl, wave, lane, xs);
        sync();  // X is in LDS
        // dQ = lower(dO V^T) K + dO X^T: A operand X[q/k index][v index], read transposed like R for dK
        walk_product<T, D, false, 0, B::KV, NQ>(tg, tv, tk, wave, lane, c > 0, [&](int db, int kc) -> V8 {
            return walk_col_frag_perm<T, D>(tl, 16 * kc, db, lane, true);
        }, acc);
        walk_store<T, D, OQ::PER>(rdq, dqs2, p.wqk, row, g, OQ::db0(wave), acc, fmap, tq, 32 * rb + l32);
        if constexpr (ACCUM) {
            prev.add_to(held);
            walk_store<T, D, OV::PER>(rdv, dvs2, p.wv, row, g, OV::db0(wave), held);
        }
        if (!(kSplitUpdate && rb == 1)) walk_update<T, D, B, false, true>(tq, tg, wave, lane, st);
        sync();  // every wave has read X and is done with the tiles
        walk_state_to_lds<T, D, B>(tl, wave, lane, st);
    }
#else
    (void)p;
#endif
}

// ---- walk_bwd_rev_kernel for q and k of 129 .. 256 columns against a v of at most 64: one reverse walk over
// both 128-column halves.  Per chunk and half h, with R_h and X_h the states of walk_bwd_rev_kernel for the half:
//   dV  += upper(K_h Q_h^T) dO + K_h R_h        (fp32 accumulators from the first half to the second, stored once)
//   dK_h = upper(V dO^T) Q_h + V R_h^T          dQ_h = lower(dO V^T) K_h + dO X_h^T
// V and dO are loaded once per chunk, where two walks of walk_bwd_rev_kernel, the second adding its part of dV to
// the first one's, load them twice, write dV twice and read it back once.
// LDS as in walk_fwd_wide_kernel: a set of (Q_h, K_h) tiles per half, two (V, dO) pairs by chunk parity, and ONE
// 16-bit state that holds R_h, then X_h, of the half at work; at the end of a half-chunk the other half's R (in
// registers throughout) is rounded into it.  Four states in registers: built for v blocks NV = 2 only.
template <typename T, int NV>
__global__ __launch_bounds__(256, 1) void walk_bwd_rev_wide_kernel(const WalkParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int D = 128, NQ = D / 32;
    static_assert(NV == 2, "R and X of both halves live in registers: two blocks per wave and state");
    using W = WalkCfg<D>;
    using V8 = typename Mma<T>::V8;
    using B = WalkExt<D, NQ, NV>;   // R, X [q/k index][v index]
    using OV = WalkOut<D, NV>;      // dV is as wide as v,
    using OQ = WalkOut<D, NQ>;      // dK and dQ as q and k
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    unsigned char *tl = smem + 8 * W::TILE;
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rb = wave % W::NRB;
    const WalkSlice sl = walk_slice(p);
    if (!sl.valid) return;
    const int b = sl.bh / p.H, h = sl.bh - b * p.H, N = p.N;
    const T *Q = static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h;
    const T *K = static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h;
    const T *V = static_cast<const T *>(p.v) + b * p.vs_b + h * p.vs_h;
    const T *G = static_cast<const T *>(p.go) + b * p.gs_b + h * p.gs_h;
    T *DQ = static_cast<T *>(p.dq) + b * p.dqs_b + h * p.dqs_h;
    T *DK = static_cast<T *>(p.dk) + b * p.dks_b + h * p.dks_h;
    T *DV = static_cast<T *>(p.dv) + b * p.dvs_b + h * p.dvs_h;
    const int qs2 = (int)p.qs_n * 2, ks2 = (int)p.ks_n * 2, vs2 = (int)p.vs_n * 2, gs2 = (int)p.gs_n * 2;
    const int dqs2 = (int)p.dqs_n * 2, dks2 = (int)p.dks_n * 2, dvs2 = (int)p.dvs_n * 2;
    const u32x4 rq0 = make_rsrc(Q, (uint32_t)((N - 1) * qs2 + p.wqk * 2));
    const u32x4 rk0 = make_rsrc(K, (uint32_t)((N - 1) * ks2 + p.wqk * 2));
    const u32x4 rq1 = make_rsrc(Q + D, (uint32_t)((N - 1) * qs2 + p.wqk2 * 2));
    const u32x4 rk1 = make_rsrc(K + D, (uint32_t)((N - 1) * ks2 + p.wqk2 * 2));
    const u32x4 rv = make_rsrc(V, (uint32_t)((N - 1) * vs2 + p.wv * 2));
    const u32x4 rg = make_rsrc(G, (uint32_t)((N - 1) * gs2 + p.wv * 2));
    const __amdgpu_buffer_rsrc_t rdq0 = __builtin_amdgcn_make_buffer_rsrc(DQ, 0, (N - 1) * dqs2 + p.wqk * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rdk0 = __builtin_amdgcn_make_buffer_rsrc(DK, 0, (N - 1) * dks2 + p.wqk * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rdq1 = __builtin_amdgcn_make_buffer_rsrc(DQ + D, 0, (N - 1) * dqs2 + p.wqk2 * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rdk1 = __builtin_amdgcn_make_buffer_rsrc(DK + D, 0, (N - 1) * dks2 + p.wqk2 * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rdv = __builtin_amdgcn_make_buffer_rsrc(DV, 0, (N - 1) * dvs2 + p.wv * 2, 0x00020000);

    f32x16 st0[W::NBW], st1[W::NBW];  // R_0, R_1
    f32x16 xs0[W::NBW], xs1[W::NBW];  // X_0, X_1
    if (p.init_is_totals) {
        const int64_t at = (int64_t)sl.bh * p.n_seg * (D * D);
        walk_sum_two<D, B>(p.init + at, p.init2 + at, sl.seg + 1, p.n_seg, wave, lane, st0, st1);
    } else {
        walk_load_init_from<D, B>(p.init, p, sl, wave, lane, st0, true);
        walk_load_init_from<D, B>(p.init2, p, sl, wave, lane, st1, true);
    }
    walk_load_end_state_from<D, B>(p.xinit, p.xtotal, p, sl, wave, lane, xs0);
    walk_load_end_state_from<D, B>(p.xinit2, p.xtotal2, p, sl, wave, lane, xs1);
    walk_state_to_lds<T, D, B>(tl, wave, lane, st0);

    auto load_half = [&](int c, auto half) {  // Q_h, K_h of chunk c to set h
        constexpr int HF = decltype(half)::value;
        const uint32_t base = lds0 + HF * 2 * W::TILE;
        walk_load_tile<D>(HF ? rq1 : rq0, base, c * W::C, qs2, HF ? p.wqk2 : p.wqk, wave, lane);
        walk_load_tile<D>(HF ? rk1 : rk0, base + W::TILE, c * W::C, ks2, HF ? p.wqk2 : p.wqk, wave, lane);
    };
    auto vg_slot = [&](int c) { return 4 + 2 * ((sl.c_hi - 1 - c) & 1); };
    auto load_vg = [&](int c) {
        const uint32_t base = lds0 + vg_slot(c) * W::TILE;
        walk_load_tile<D>(rv, base, c * W::C, vs2, p.wv, wave, lane);
        walk_load_tile<D>(rg, base + W::TILE, c * W::C, gs2, p.wv, wave, lane);
    };
    auto sync = [&]() {  // this wave's LDS accesses are done; then every wave's
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    // A operands of the state products: R^T[v index][q/k index] is the LDS copy as it is (dV); R and X
    // [q/k index][v index] are the copy read transposed (dK, dQ)
    auto rows_of_state = [&](int db, int kc) -> V8 { return walk_row_frag<T, D>(tl, 32 * db + walk_e_lane(l32), kc, g); };
    auto cols_of_state = [&](int db, int kc) -> V8 { return walk_col_frag_perm<T, D>(tl, 16 * kc, db, lane, true); };
    load_half(sl.c_hi - 1, std::integral_constant<int, 0>{});
    load_vg(sl.c_hi - 1);
#pragma unroll 1
    for (int c = sl.c_hi - 1; c >= sl.c_lo; --c) {
        unsigned char *tv = smem + vg_slot(c) * W::TILE, *tg = tv + W::TILE;
        const int row = c * W::C + 32 * rb + l32;
        const bool later = c + 1 < p.n_chunks;  // chunks after this one exist: R is not identically zero
        f32x16 dvacc[W::DBW];
        auto half_chunk = [&](auto half, f32x16 (&st)[W::NBW], f32x16 (&xs)[W::NBW], f32x16 (&st_next)[W::NBW]) {
            constexpr int HF = decltype(half)::value;
            unsigned char *tq = smem + HF * 2 * W::TILE, *tk = tq + W::TILE;
            // (every wave has left the barrier that ended the reads of the set loaded next, one half-chunk ago.)
            // This wave's loads of the half-chunk have landed when at most the loads issued after them are
            // outstanding; the stores of the half-chunk before were issued before those.
            if constexpr (HF == 0) {
                load_half(c, std::integral_constant<int, 1>{});
                wait_vm<2 * W::NI>();
            } else {
                if (c > sl.c_lo) {
                    load_half(c - 1, std::integral_constant<int, 0>{});
                    load_vg(c - 1);  // (to the slots of the chunk after this one)
                    wait_vm<4 * W::NI>();
                } else {
                    wait_vm<0>();
                }
            }
            sync();  // the tiles have landed, R_h is in LDS
            walk_update<T, D, B, true, true>(tk, tv, wave, lane, xs);  // X_h: now the sum over the chunks before this one
            walk_product<T, D, true, 0, B::KQ, NV, HF != 0>(tk, tq, tg, wave, lane, later, rows_of_state, dvacc);
            f32x16 acc[W::DBW];
            walk_product<T, D, true, 0, B::KV, NQ>(tv, tg, tq, wave, lane, later, cols_of_state, acc);
            walk_store<T, D, OQ::PER>(HF ? rdk1 : rdk0, dks2, HF ? p.wqk2 : p.wqk, row, g, OQ::db0(wave), acc);
            sync();  // every wave has read R_h
            // (X stays in its accumulation registers up to here: without this the copies that the rounding
            // below reads are made right after the update and occupy registers through both products)
            asm volatile("" : "+a"(xs[0]), "+a"(xs[1]));
            walk_state_to_lds<T, D, B>(tl, wave, lane, xs);
            sync();  // X_h is in LDS
            walk_product<T, D, false, 0, B::KV, NQ>(tg, tv, tk, wave, lane, c > 0, cols_of_state, acc);
            walk_store<T, D, OQ::PER>(HF ? rdq1 : rdq0, dqs2, HF ? p.wqk2 : p.wqk, row, g, OQ::db0(wave), acc);
            if constexpr (HF != 0) walk_store<T, D, OV::PER>(rdv, dvs2, p.wv, row, g, OV::db0(wave), dvacc);
            walk_update<T, D, B, false, true>(tq, tg, wave, lane, st);  // R_h += Q_h^T dO
            sync();  // every wave has read X_h and is done with this half's tiles
            walk_state_to_lds<T, D, B>(tl, wave, lane, st_next);
        };
        half_chunk(std::integral_constant<int, 0>{}, st0, xs0, st1);
        half_chunk(std::integral_constant<int, 1>{}, st1, xs1, st0);
    }
#else
    (void)p;
#endif
}

// ---- segment totals: totals[bh][seg] = sum over the segment's rows of Y^T Z, fp32 [D][D]
struct WalkTotalsParams {
    const void *y, *z;
    int64_t ys_b, ys_h, ys_n, zs_b, zs_h, zs_n;
    int32_t H, N, BH, dy, dz;
    int32_t n_chunks, seg_chunks, n_seg;
    int32_t seg_lo, seg_hi;  // only segments seg_lo .. seg_hi - 1 are needed (the others' totals stay unwritten)
    float *totals;
    // two segments: only the total of segment seg_lo is needed, as the other segment's entry state.
    // The kernel writes it in the layout the walks read (see walk_load_init) -- `totals` is where
    // the entry states go -- and no scan follows.
    int32_t direct;
    // feature map on load: Y holds the argument of the map; every Y tile is mapped in LDS as it lands
    // and the mapped rows are written to ymap_out (Y's shape, element strides yo_*).  0: none.
    int32_t map_y;
    void *ymap_out;
    int64_t yo_b, yo_h, yo_n;
    // A second Y operand of the same layout against the same Z, in the same launch: the other 128-column half
    // of a wide q / k, whose totals go to `totals2`.  Null: none.  (Without a feature map.)  Grid y = 1 takes
    // it, or -- the kernel variant with BOTH -- every workgroup takes both operands.
    const void *y2;
    int32_t dy2;
    float *totals2;
};

constexpr int walk_totals_sets(int D) { return D == 128 ? 4 : 2; }  // sets of (Y, Z) tiles in LDS

// BOTH (D = 128, NV = 2): the launch's two Y operands (WalkTotalsParams::y2) in ONE workgroup -- three sets of
// (Y, Y2, Z) tiles, a state per operand -- so that Z is loaded once for the two; otherwise grid y picks the operand.
template <typename T, int D, int NQ = D / 32, int NV = D / 32, bool BOTH = false>
__global__ __launch_bounds__(256, BOTH ? 1 : 2) void walk_totals_kernel(const WalkTotalsParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    using W = WalkCfg<D>;
    static_assert(!BOTH || (D == 128 && NV == 2), "two states per wave: built for the narrow v side of D = 128");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = blockIdx.x, xcd = wg & 7, slot = wg >> 3;
    const int hl = slot / p.n_seg, bh = hl * 8 + xcd;
    int seg = slot - hl * p.n_seg;
    if (bh >= p.BH) return;
    const bool second = !BOTH && blockIdx.y != 0;  // (the launch's second Y operand: see WalkTotalsParams::y2)
    const int dy = second ? p.dy2 : p.dy;
    int64_t out_at;
    int c_lo, c_hi;
    if (p.direct) {
        // both workgroups of a (b, h) at work: half of the needed segment's chunks each (with a feature map
        // every row has to be visited: the needed segment's workgroup forms its total alone, the other one
        // maps its own segment's rows and hands in zeros)
        const int needed = p.seg_lo, part = seg != needed;
        out_at = ((int64_t)bh * 2 + part) * (D * D);
        c_lo = seg * p.seg_chunks;
        c_hi = c_lo + p.seg_chunks < p.n_chunks ? c_lo + p.seg_chunks : p.n_chunks;
        if (!p.map_y) {
            const int n_lo = needed * p.seg_chunks;
            const int n_hi = n_lo + p.seg_chunks < p.n_chunks ? n_lo + p.seg_chunks : p.n_chunks;
            const int mid = n_lo + (n_hi - n_lo + 1) / 2;
            c_lo = part ? mid : n_lo, c_hi = part ? n_hi : mid;
        }
    } else {
        if (seg < p.seg_lo || seg >= p.seg_hi) return;
        out_at = ((int64_t)bh * p.n_seg + seg) * (D * D);
        c_lo = seg * p.seg_chunks;
        c_hi = c_lo + p.seg_chunks < p.n_chunks ? c_lo + p.seg_chunks : p.n_chunks;
    }
    float *const out = (second ? p.totals2 : p.totals) + out_at;
    float *const out2 = BOTH ? p.totals2 + out_at : nullptr;
    if (c_lo >= c_hi) {  // nothing to add up (a segment beyond the end of the sequence, the second half of one chunk)
        for (int i = tid; i < D * D; i += 256) {
            out[i] = 0.f;
            if constexpr (BOTH) out2[i] = 0.f;
        }
        return;
    }
    const bool discard = p.direct && p.map_y && seg != p.seg_lo;  // (visited for the map only)
    const int b = bh / p.H, h = bh - b * p.H, N = p.N;
    const T *Y = static_cast<const T *>(second ? p.y2 : p.y) + b * p.ys_b + h * p.ys_h;
    const T *Y2 = static_cast<const T *>(BOTH ? p.y2 : p.y) + b * p.ys_b + h * p.ys_h;
    const T *Z = static_cast<const T *>(p.z) + b * p.zs_b + h * p.zs_h;
    const int ys2 = (int)p.ys_n * 2, zs2 = (int)p.zs_n * 2;
    const u32x4 ry = make_rsrc(Y, (uint32_t)((N - 1) * ys2 + dy * 2));
    const u32x4 ry2 = make_rsrc(Y2, (uint32_t)((N - 1) * ys2 + (BOTH ? p.dy2 : dy) * 2));
    const u32x4 rz = make_rsrc(Z, (uint32_t)((N - 1) * zs2 + p.dz * 2));
    using B = WalkExt<D, NQ, NV>;  // (blocks outside it stay unwritten: no walk of the same extent reads them)
    f32x16 st[W::NBW], st2[W::NBW];
#pragma unroll
    for (int i = 0; i < W::NBW; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) st[i][v] = 0.f, st2[i][v] = 0.f;
    // SETS sets of tiles.  Two (two workgroups per CU): the loads of chunk c + 1 are in flight while
    // chunk c is multiplied.  More (D = 128, where the grid has at most one workgroup per CU and a
    // workgroup's own chain load -> barrier -> product bounds its rate): SETS - 1 chunks in flight.
    constexpr int SETS = BOTH ? 3 : walk_totals_sets(D), TPS = BOTH ? 3 : 2;  // tiles per set: Y, (Y2,) Z
    auto load_chunk = [&](int c, int set) {
        const uint32_t base = lds0 + set * TPS * W::TILE;
        walk_load_tile<D>(ry, base, c * W::C, ys2, dy, wave, lane);
        if constexpr (BOTH) walk_load_tile<D>(ry2, base + W::TILE, c * W::C, ys2, p.dy2, wave, lane);
        walk_load_tile<D>(rz, base + (TPS - 1) * W::TILE, c * W::C, zs2, p.dz, wave, lane);
    };
    auto map_tile = [&](unsigned char *ty, int c) {
        walk_map_tile<T, D>(ty, p.map_y, c * W::C, N, dy, static_cast<T *>(p.ymap_out) + b * p.yo_b + h * p.yo_h,
                            p.yo_n, tid);
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the rewritten tile is in LDS
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    if constexpr (SETS == 2) {
        load_chunk(c_lo, 0);
#pragma unroll 1
        for (int c = c_lo; c < c_hi; ++c) {
            const int buf = (c - c_lo) & 1;
            unsigned char *ty = smem + buf * 2 * W::TILE, *tz = ty + W::TILE;
            const bool more = c + 1 < c_hi;
            if (more) load_chunk(c + 1, buf ^ 1);  // (every wave has left the barrier that ended the reads of that set)
            // this wave's loads of chunk c have landed: only those of chunk c + 1 may still be in flight
            // (the mapped rows' stores of a feature map share the counter: then everything is awaited)
            if (more && !p.map_y)
                wait_vm<2 * W::NI>();
            else
                wait_vm<0>();
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (p.map_y) map_tile(ty, c);
            walk_update<T, D, B>(ty, tz, wave, lane, st);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0xc07f);  // this wave's LDS reads of the set are done
            __builtin_amdgcn_s_barrier();
        }
    } else {
        static_assert(SETS == 3 || SETS == 4, "the waits below count up to two chunks behind the awaited one");
#pragma unroll
        for (int i = 0; i < SETS - 1; ++i)
            if (c_lo + i < c_hi) load_chunk(c_lo + i, i);
        int set = 0;
#pragma unroll 1
        for (int c = c_lo; c < c_hi; ++c) {
            unsigned char *ty = smem + set * TPS * W::TILE, *tz = ty + (TPS - 1) * W::TILE;
            // this wave's loads of chunk c have landed: those of up to SETS - 2 later chunks may still be in
            // flight (the mapped rows' stores of a feature map share the counter: then everything is awaited)
            const int behind = c_hi - 1 - c;
            if (p.map_y || behind == 0)
                wait_vm<0>();
            else if (behind == 1 || SETS == 3)
                wait_vm<TPS * W::NI>();
            else
                wait_vm<2 * TPS * W::NI>();
            __builtin_amdgcn_s_waitcnt(0xc07f);  // this wave's LDS reads of the chunk before are done
            __builtin_amdgcn_s_barrier();        // ... and so are every wave's: its set can be loaded over
            asm volatile("" ::: "memory");
            if (c + SETS - 1 < c_hi) load_chunk(c + SETS - 1, (set + SETS - 1) % SETS);
            if (p.map_y) map_tile(ty, c);
            walk_update<T, D, B>(ty, tz, wave, lane, st);
            if constexpr (BOTH) walk_update<T, D, B>(ty + W::TILE, tz, wave, lane, st2);
            asm volatile("" ::: "memory");
            set = (set + 1) % SETS;
        }
    }
#pragma unroll
    for (int i = 0; i < B::SLOTS; ++i)
        if (B::valid(wave, i)) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int at = (32 * B::dbk(wave, i) + 8 * (v / 4) + 4 * g + (v % 4)) * D + 32 * B::eb(wave) + l32;
                out[at] = discard ? 0.f : st[i][v];
                if constexpr (BOTH) out2[at] = st2[i][v];
            }
        }
#else
    (void)p;
#endif
}

// Entry states of the walk's segments from the segments' totals: entry[bh][s][e] = sum of
// totals[bh][f][e] over f < s (reverse == 0) or f > s (reverse != 0).  Only the totals under those
// sums are read.  entry may be totals (a thread reads an element before it writes it).  One thread
// per pair of elements; the loads of up to sixteen segments are issued together (a chain of
// dependent loads would cost a memory latency each).
// `cols`: only the first `cols` columns of every row of the D-wide states are summed (the totals
// kernel built for a narrow v side writes no others, and no walk of that extent reads them).
// (a template only so that the header can be included by several translation units)
// grid y = 1 scans a second pair of buffers of the same shape (totals_b, entry_b; the other half of a wide q / k).
template <int kUnused = 0>
__global__ __launch_bounds__(256) void walk_scan_kernel(const float *totals, float *entry, int n_seg, int E,
                                                        int64_t total2, int reverse, int D, int cols,
                                                        const float *totals_b, float *entry_b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const int64_t i2 = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i2 >= total2) return;
    if (blockIdx.y != 0) totals = totals_b, entry = entry_b;
    const int half = cols / 2;
    const int64_t per_bh = (int64_t)(E / D) * half, bh = i2 / per_bh, r = i2 - bh * per_bh;
    const int64_t e = (r / half) * D + 2 * (r % half);
    const float *pt = totals + bh * n_seg * E + e;
    float *pe = entry + bh * n_seg * E + e;
    const int64_t step = reverse ? -(int64_t)E : (int64_t)E;
    if (reverse) pt += (int64_t)(n_seg - 1) * E, pe += (int64_t)(n_seg - 1) * E;
    f32x2 run = {0.f, 0.f};
    int s = 0;
    auto batch = [&](auto nn) {
        constexpr int NB = decltype(nn)::value;
        for (; s + NB <= n_seg - 1; s += NB) {
            f32x2 t[NB];
#pragma unroll
            for (int u = 0; u < NB; ++u) t[u] = *reinterpret_cast<const f32x2 *>(pt + u * step);
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                *reinterpret_cast<f32x2 *>(pe + u * step) = run;
                run += t[u];
            }
            pt += NB * step, pe += NB * step;
        }
    };
    batch(std::integral_constant<int, 16>{});
    batch(std::integral_constant<int, 4>{});
    batch(std::integral_constant<int, 1>{});
    *reinterpret_cast<f32x2 *>(pe) = run;  // the last segment in walking order: its own total is not needed
}

// ---- per-chunk column sums for the normaliser's running vectors: out[bh][c][col] = sum over the
// rows of chunk c of w[row] y[row][col] (w null: plain sums); fp32.  A scan over the chunks
// (walk_vec_scan_kernel) then gives zc (y = k, prefix) or rc (y = q, w = dn, suffix).
struct WalkVecParams {
    const void *y;
    int64_t ys_b, ys_h, ys_n;
    const float *w;  // [BH][N] or null
    int32_t H, N, width, n_chunks;
    float *out;      // [BH][n_chunks][D]
};

template <typename T, int D>
__global__ __launch_bounds__(256) void walk_vec_sums_kernel(const WalkVecParams p) {
    using W = WalkCfg<D>;
    using V8 = typename Mma<T>::V8;
    constexpr int SLOTS = 256 / W::CR;  // rows visited at a time
    __shared__ float part[SLOTS][D];
    const int tid = threadIdx.x, pos = tid % W::CR, slot = tid / W::CR;
    const int c = blockIdx.x, bh = blockIdx.y, b = bh / p.H, h = bh - b * p.H;
    const T *Y = static_cast<const T *>(p.y) + b * p.ys_b + h * p.ys_h;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    if (pos * 8 < p.width) {
#pragma unroll 4
        for (int r = slot; r < W::C; r += SLOTS) {
            const int row = c * W::C + r;
            if (row < p.N) {
                const V8 y = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4 *>(Y + (int64_t)row * p.ys_n + pos * 8));
                const float w = p.w ? p.w[(int64_t)bh * p.N + row] : 1.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] += w * static_cast<float>(y[e]);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) part[slot][pos * 8 + e] = acc[e];
    __syncthreads();
    if (tid < D) {
        float t = 0.f;
#pragma unroll
        for (int u = 0; u < SLOTS; ++u) t += part[u][tid];
        p.out[((int64_t)bh * p.n_chunks + c) * D + tid] = t;
    }
}

// ---- exclusive prefix (reverse: suffix) sums over the chunks of the vectors above, in place:
// v[bh][c][col] <- sum of v[bh][c'][col] over c' < c (c' > c).  There are few columns and many
// chunks, so the chunks of a (b, h) are split over sixteen thread groups: each adds up its range,
// the ranges' sums are scanned in LDS, and each group writes its range's running sums.
// (a template only so that the header can be included by several translation units)
template <int kUnused = 0>
__global__ __launch_bounds__(256) void walk_vec_scan_kernel(float *v, int n_chunks, int D, int reverse) {
    __shared__ float part[16][16];
    const int j = threadIdx.x & 15, grp = threadIdx.x >> 4;  // column within the block's 16, range of chunks
    const int bh = blockIdx.y, col = blockIdx.x * 16 + j;
    const int per = (n_chunks + 15) / 16;
    float *base = v + (int64_t)bh * n_chunks * D + col;
    // walking order: position t = 0 .. n_chunks - 1 is chunk t, or chunk n_chunks - 1 - t in reverse
    const int t0 = grp * per, t1 = t0 + per < n_chunks ? t0 + per : n_chunks;
    auto chunk_of = [&](int t) { return reverse ? n_chunks - 1 - t : t; };
    float sum = 0.f;
    for (int t = t0; t < t1; t += 8) {
        float x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = t + u < t1 ? base[(int64_t)chunk_of(t + u) * D] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += x[u];
    }
    part[grp][j] = sum;
    __syncthreads();
    float run = 0.f;
    for (int g2 = 0; g2 < grp; ++g2) run += part[g2][j];
    for (int t = t0; t < t1; t += 8) {
        float x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = t + u < t1 ? base[(int64_t)chunk_of(t + u) * D] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (t + u < t1) {
                base[(int64_t)chunk_of(t + u) * D] = run;
                run += x[u];
            }
    }
}

inline hipError_t launch_walk_vec_scan(float *v, int64_t BH, int n_chunks, int D, int reverse, hipStream_t stream) {
    if (BH > 65535 || D % 16 != 0) return hipErrorInvalidConfiguration;
    return launch_kernel<walk_vec_scan_kernel<0>>(dim3((unsigned)(D / 16), (unsigned)BH), dim3(256), 0, stream, v, n_chunks,
                         D, reverse);
}

template <typename T, int D>
hipError_t launch_walk_vec_sums(const WalkVecParams &p, int64_t BH, hipStream_t stream) {
    if (BH > 65535) return hipErrorInvalidConfiguration;
    return launch_kernel<walk_vec_sums_kernel<T, D>>(dim3((unsigned)p.n_chunks, (unsigned)BH), dim3(256), 0, stream, p);
}

// columns of the D x D totals that walk_totals_kernel writes for operands of true widths dy, dz (the
// variant without the padding blocks of a narrow z leaves the others unwritten)
inline int walk_totals_cols(int D, int dy, int dz) { return D == 128 && dy > 64 && dz <= 64 ? 64 : D; }

template <typename T, int D>
hipError_t launch_walk_totals(const WalkTotalsParams &p, hipStream_t stream) {
    const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * p.n_seg;
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    constexpr int smem = walk_totals_sets(D) * 2 * WalkCfg<D>::TILE;
    if (p.direct && (p.n_seg != 2 || p.seg_lo < 0 || p.seg_lo > 1)) return hipErrorInvalidValue;
    // (a second operand runs the same kernel variant: the caller pairs operands of one kind only)
    if (p.y2 && (p.map_y || !p.totals2 || walk_totals_cols(D, p.dy2, p.dz) != walk_totals_cols(D, p.dy, p.dz)))
        return hipErrorInvalidValue;
    const dim3 g((unsigned)grid, p.y2 ? 2u : 1u);
    if constexpr (D == 128) {
        if (p.y2 && walk_totals_cols(D, p.dy, p.dz) == 64) {  // ... and both operands in one workgroup: z loaded once
            constexpr auto kern = walk_totals_kernel<T, D, 4, 2, true>;
            constexpr int smem_both = 3 * 3 * WalkCfg<D>::TILE;
            if (hipError_t e = ensure_dynamic_lds<kern>(smem_both)) return e;
            return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem_both, stream, p);
        }
        if (walk_totals_cols(D, p.dy, p.dz) == 64) {  // z of at most 64 true columns: the state's other v blocks hold zeros
            constexpr auto kern = walk_totals_kernel<T, D, 4, 2>;
            if (hipError_t e = ensure_dynamic_lds<kern>(smem)) return e;
            return launch_kernel<kern>(g, dim3(256), smem, stream, p);
        }
    }
    constexpr auto kern = walk_totals_kernel<T, D>;
    if (hipError_t e = ensure_dynamic_lds<kern>(smem)) return e;
    return launch_kernel<kern>(g, dim3(256), smem, stream, p);
}

inline hipError_t launch_walk_scan(const float *totals, float *entry, int64_t BH, int n_seg, int D, int cols,
                                   int reverse, hipStream_t stream, const float *totals_b = nullptr,
                                   float *entry_b = nullptr) {
    const int E = D * D;
    const int64_t total2 = BH * D * (cols / 2);
    if (n_seg < 1 || cols < 2 || cols > D || cols % 2 || (totals_b != nullptr) != (entry_b != nullptr))
        return hipErrorInvalidValue;
    return launch_kernel<walk_scan_kernel<0>>(dim3((unsigned)((total2 + 255) / 256), totals_b ? 2u : 1u), dim3(256), 0,
                                              stream, totals, entry, n_seg, E, total2, reverse, D, cols, totals_b, entry_b);
}

template <auto kern>
hipError_t launch_walk_kernel(int64_t grid, int smem, const WalkParams &p, hipStream_t stream) {
    if (hipError_t e = ensure_dynamic_lds<kern>(smem)) return e;
    return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem, stream, p);
}

template <typename T, int D>
hipError_t launch_walk_fwd(const WalkParams &p, hipStream_t stream) {
    const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * p.n_seg;
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    constexpr bool kDouble = D > 64;  // (the plan's workgroup count must match: one per CU when double)
    constexpr int smem = (kDouble ? 6 : 3) * WalkCfg<D>::TILE + WalkCfg<D>::STATE;
    const bool fm = p.fmap || p.slope_y;
    // (segment totals in place of entry states: the D = 128 walks, by the flag; below that by the number of segments)
    if (p.init_is_totals && (D != 128 || p.n_seg < 3 || !p.init)) return hipErrorInvalidValue;
    if (p.entry_out && (!p.init_is_totals || fm || p.denom || p.dn)) return hipErrorInvalidValue;
    if (p.denom || p.dn) {  // the normaliser's terms: its vectors live behind the state
        if (!p.zc || p.accumulate) return hipErrorInvalidValue;
        constexpr int smem_n = smem + (kDouble ? 2 : 1) * WalkCfg<D>::VEC;
        if (p.denom)
            return fm ? launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 1, true>>(grid, smem_n, p, stream)
                      : launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 1, false>>(grid, smem_n, p, stream);
        return fm ? launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 2, true>>(grid, smem_n, p, stream)
                  : launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 2, false>>(grid, smem_n, p, stream);
    }
    if (fm) return p.accumulate ? hipErrorNotSupported : launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 0, true>>(grid, smem, p, stream);
    if constexpr (D == 128) {
        // operands of at most 64 true columns on one side (the halves of a wide q / k against a narrow v):
        // the kernels that leave out the blocks of padding
        if (p.wqk > 64 && p.wv <= 64)
            return p.accumulate ? launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 0, false, 4, 2, true>>(grid, smem, p, stream)
                                : launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 0, false, 4, 2>>(grid, smem, p, stream);
        if (p.wqk <= 64 && p.wv > 64)
            return p.accumulate ? launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 0, false, 2, 4, true>>(grid, smem, p, stream)
                                : launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 0, false, 2, 4>>(grid, smem, p, stream);
        if (p.accumulate) return launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 0, false, 4, 4, true>>(grid, smem, p, stream);
    }
    if (p.accumulate) return hipErrorNotSupported;
    return launch_walk_kernel<walk_fwd_kernel<T, D, kDouble, 0, false>>(grid, smem, p, stream);
}

template <typename T>
hipError_t launch_walk_fwd_wide(const WalkParams &p, hipStream_t stream) {
    using W = WalkCfg<128>;
    const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * p.n_seg;
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    if (p.wqk != 128 || p.wqk2 < 1 || p.wqk2 > 128 || p.wv < 1 || p.wv > 128 || p.fmap || p.slope_y || p.denom || p.dn ||
        p.accumulate || p.init_transposed || (p.n_seg > 1 && (!p.init || !p.init2)) || (p.total_out && !p.total_out2) ||
        (p.init_is_totals && (p.n_seg < 3 || !p.init || !p.init2)) ||
        (p.entry_out != nullptr) != (p.entry_out2 != nullptr) || (p.entry_out && !p.init_is_totals))
        return hipErrorInvalidValue;
    constexpr int smem = 6 * W::TILE + W::STATE;  // two sets of (Q_h, K_h), two V tiles, one state
    if (p.wv <= 64) return launch_walk_kernel<walk_fwd_wide_kernel<T, 2>>(grid, smem, p, stream);
    return launch_walk_kernel<walk_fwd_wide_kernel<T, 4>>(grid, smem, p, stream);
}

template <typename T, int D>
hipError_t launch_walk_bwd(const WalkParams &p, hipStream_t stream) {
    const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * p.n_seg;
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    constexpr int smem = 4 * WalkCfg<D>::TILE + WalkCfg<D>::STATE;
    if (p.dn) {
        if (!p.zc || !p.rc) return hipErrorInvalidValue;
        constexpr auto kern = walk_bwd_kernel<T, D, true>;
        constexpr int smem_n = smem + WalkCfg<D>::VEC;
        if (hipError_t e = ensure_dynamic_lds<kern>(smem_n)) return e;
        return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem_n, stream, p);
    }
    if (!p.xtotal || (p.n_seg > 1 && !p.xinit)) return hipErrorInvalidValue;
    constexpr auto kern = walk_bwd_kernel<T, D, false>;
    constexpr int smem_x = smem + WalkCfg<D>::STATE;  // X's copy beside R's
    if (hipError_t e = ensure_dynamic_lds<kern>(smem_x)) return e;
    return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem_x, stream, p);
}

template <typename T, int D>
hipError_t launch_walk_dkdv(const WalkParams &p, hipStream_t stream) {
    const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * p.n_seg;
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    constexpr int smem = 8 * WalkCfg<D>::TILE + WalkCfg<D>::STATE;
    static_assert(smem <= 160 * 1024, "two sets of tiles and the state must fit the LDS of a CU");
    if (p.dn) {
        if (!p.rc) return hipErrorInvalidValue;
        constexpr auto kern = walk_dkdv_kernel<T, D, true>;
        if (hipError_t e = ensure_dynamic_lds<kern>(smem)) return e;
        return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem, stream, p);
    }
    if constexpr (D == 128) {
        if (!p.fmap && p.wqk > 64 && p.wv <= 64) {
            constexpr auto kern = walk_dkdv_kernel<T, D, false, 4, 2>;
            if (hipError_t e = ensure_dynamic_lds<kern>(smem)) return e;
            return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem, stream, p);
        }
    }
    constexpr auto kern = walk_dkdv_kernel<T, D, false>;
    if (hipError_t e = ensure_dynamic_lds<kern>(smem)) return e;
    return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem, stream, p);
}

template <typename T, int D>
hipError_t launch_walk_bwd_rev(const WalkParams &p, hipStream_t stream) {
    const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * p.n_seg;
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    if (!p.xtotal || (p.n_seg > 1 && !p.xinit)) return hipErrorInvalidValue;
    if (p.entry_out || (p.init_is_totals && (p.n_seg < 3 || !p.init))) return hipErrorInvalidValue;
    constexpr int smem = 8 * WalkCfg<D>::TILE + WalkCfg<D>::STATE;
    static_assert(smem <= 160 * 1024, "two sets of tiles and the state must fit the LDS of a CU");
    if constexpr (D == 128) {  // a half of a wide q / k against a narrow v: without the blocks of padding
        if (!p.fmap && p.wqk > 64 && p.wv <= 64)
            return p.accumulate ? launch_walk_kernel<walk_bwd_rev_kernel<T, D, 4, 2, true>>(grid, smem, p, stream)
                                : launch_walk_kernel<walk_bwd_rev_kernel<T, D, 4, 2>>(grid, smem, p, stream);
    }
    if (p.fmap) {
        if (p.accumulate) return hipErrorNotSupported;
        return launch_walk_kernel<walk_bwd_rev_kernel<T, D, D / 32, D / 32, false, true>>(grid, smem, p, stream);
    }
    if (p.accumulate) return launch_walk_kernel<walk_bwd_rev_kernel<T, D, D / 32, D / 32, true>>(grid, smem, p, stream);
    return launch_walk_kernel<walk_bwd_rev_kernel<T, D>>(grid, smem, p, stream);
}

template <typename T>
hipError_t launch_walk_bwd_rev_wide(const WalkParams &p, hipStream_t stream) {
    using W = WalkCfg<128>;
    const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * p.n_seg;
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    if (p.wqk != 128 || p.wqk2 < 1 || p.wqk2 > 128 || p.wv < 1 || p.wv > 64) return hipErrorNotSupported;
    if (p.fmap || p.dn || p.accumulate || p.init_transposed || !p.xtotal || !p.xtotal2 || p.entry_out || p.entry_out2 ||
        (p.n_seg > 1 && (!p.init || !p.init2 || !p.xinit || !p.xinit2)) || (p.init_is_totals && p.n_seg < 3))
        return hipErrorInvalidValue;
    constexpr int smem = 8 * W::TILE + W::STATE;  // two sets of (Q_h, K_h), two of (V, dO), one state
    static_assert(smem <= 160 * 1024, "the tiles and the state must fit the LDS of a CU");
    return launch_walk_kernel<walk_bwd_rev_wide_kernel<T, 2>>(grid, smem, p, stream);
}


}  // namespace fla

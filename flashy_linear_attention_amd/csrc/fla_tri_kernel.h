// Out = mask(X Y^T) Z on gfx950 MFMA: the one kernel behind forward and all
// three gradients of causal linear attention.
//
//   X, Y : (B, H, N, DC)   Z, Out : (B, H, N, DO)   16-bit storage, fp32 accumulate
//   mask : lower triangle (row >= col) or upper triangle (row <= col), diagonal kept
//
// Work decomposition
//   * One workgroup (4 wavefronts of 64 lanes) owns BM = 4*MW consecutive rows
//     of X for one (b, h) and walks the BN = 64 row tiles of Y and Z that the
//     mask leaves non-zero.
//   * Each wavefront keeps its MW rows of X in registers as MFMA operands for
//     the whole walk, and its MW x DO slice of Out in fp32 accumulators.
//   * Y and Z tiles are staged global -> registers -> LDS, double buffered, one
//     barrier per tile.
//   * Per 32-row sub-tile of Y/Z the wavefront computes S^T = Y_sub X_w^T with
//     v_mfma_f32_32x32x16 (A operand = rows of Y read from LDS with
//     ds_read_b128, B operand = resident X fragments).  In the accumulator
//     layout of that instruction lane l holds column (l % 32) and rows
//     8*(v/4) + 4*(l/32) + v%4 -- which is exactly an A operand (row = l % 32,
//     eight k-slots) of the second product Out += P Z once rounded to 16 bit,
//     provided the k-slots of the Z operand are taken in the same permuted
//     order.  So P never travels through LDS.
//   * The Z operand needs eight rows of one Z column per lane; Z sits row-major
//     in LDS, so it is fetched with ds_read_b64_tr_b16 (a 4x16 transposing
//     read inside each group of 16 lanes: lane i supplies the address of row
//     i/4, columns 4*(i%4)..+3 and receives rows 0..3 of column i).
//   * Workgroup -> (head, tile) decoding keeps all tiles of a head on one XCD
//     (workgroups are handed to the 8 XCDs round-robin by linear id), heads in
//     sequence and heavy tiles first, so that the Y/Z re-reads of a head hit
//     that XCD's L2.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fla_launch.h"

namespace fla {

struct TriParams {
    const void *x, *y, *z;
    void *out;
    int64_t xs_b, xs_h, xs_n;  // element strides; the innermost stride is 1
    int64_t ys_b, ys_h, ys_n;
    int64_t zs_b, zs_h, zs_n;
    int64_t os_b, os_h, os_n;
    int32_t H, N, BH;
    int32_t dc, dout;  // actual widths (<= DC, DO of the instantiation)
    int32_t upper;     // 0: keep row >= col, 1: keep row <= col
    int32_t n_tiles;   // ceil(N / BM), filled by the launcher
    int32_t single;    // fast path: one row tile per workgroup instead of a balanced pair (launcher's choice)
    int32_t vec_x, vec_y, vec_z;  // 1: rows are 16-byte aligned and width % 8 == 0
    int32_t vec_out;              // same for the output
    // Chunked evaluation (fast path only): when non-null, each workgroup computes only the
    // diagonal BM x BM block of its row tile and adds X_tile . S, where S is the 16-bit sum of
    // Y_c^T Z_c over the chunks before (lower) / after (upper) the tile, stored transposed as
    // state[(bh * n_tiles + tile)][DO][DC] with the padded DO, DC of the instantiation.
    const void *state;
    // 1: `state` holds the transpose instead, [DC][DO] per (bh, tile) -- the running state of the
    // product with Y and Z exchanged, shared rather than recomputed (square instantiations only)
    int32_t state_transposed;
    // Normalised output (quadratic fast path only): when non-null, each row of Out is divided by
    // n = (sum of its masked scores, in fp32 before rounding) + eps, and n is written here as
    // fp32, contiguous (B H, N).
    float *denom;
    float eps;
    // Polynomial score map (quadratic fast path, contraction width <= 64): when poly_on != 0 every
    // score u = x . y is replaced by poly[0] + poly[1] u + poly[2] u^2 before masking and rounding --
    // causal linear attention with a second-order Taylor feature map, the features never built.
    // poly_on == 2: dual-score walk (32-wide outputs only).  X and Y carry two operands side by side,
    // columns [0, DC/2) and [DC/2, DC/2 + 32) of the instantiation's padded width DC; the score is
    // u1 (poly[0] + poly[1] u2 + poly[2] u2^2).  poly_on == 3: the same with the second operand in the
    // last 32 columns, [DC - 32, DC).
    float poly[3];
    int32_t poly_on;
    // Feature map on load (chunk-wise fast path only; fla_feature.h).  map_x != 0: X holds the
    // argument x of the feature map phi; every element is replaced by phi(x) as the rows arrive
    // (columns beyond the true width stay zero), and the mapped rows are also written to
    // `xmap_out` (X's shape, element strides xo_*) for later passes.  `omap`, when non-null, is a
    // tensor of Out's shape (element strides ms_*) holding y = phi(x): each output element is
    // multiplied by phi'(x) computed from y, map_out naming phi -- the chain rule of a gradient with
    // respect to the argument of phi.
    int32_t map_x, map_out;
    void *xmap_out;
    int64_t xo_b, xo_h, xo_n;
    const void *omap;
    int64_t ms_b, ms_h, ms_n;
};

// Up to three products of identical shape in one launch (grid y selects the product): the
// backward's dQ, dV and dK.  Workgroups of the next product fill the CUs the previous one's
// tail leaves idle.
struct TriBatch {
    TriParams p[3];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

template <typename T>
struct Mma;

template <>
struct Mma<__bf16> {
    using V8 = bf16x8;
    static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    // c += a b with c held in accumulation registers throughout (a running sum that only MFMAs and
    // an occasional read touch leaves the architectural registers to the rest of the kernel).  The
    // s_nop covers a register copy the compiler may have placed right in front: it does not look
    // inside the statement for the wait states such a copy needs before an MFMA reads its target.
    static __device__ __forceinline__ void mma_acc(V8 a, V8 b, f32x16 &c) {
        asm("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};

template <>
struct Mma<_Float16> {
    using V8 = f16x8;
    static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma_acc(V8 a, V8 b, f32x16 &c) {
        asm("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};

// Eight consecutive 16-bit elements of one row, zero beyond `dlim` columns or
// when the row is out of range.
template <typename T>
__device__ __forceinline__ u32x4 load8(const T *row, bool row_ok, int col, int dlim, bool vec) {
    u32x4 r = {0u, 0u, 0u, 0u};
    if (row_ok) {
        if (vec) {
            if (col < dlim) r = *reinterpret_cast<const u32x4 *>(row + col);
        } else {
            const unsigned short *e = reinterpret_cast<const unsigned short *>(row);
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                uint32_t lo = (col + 2 * x < dlim) ? e[col + 2 * x] : 0u;
                uint32_t hi = (col + 2 * x + 1 < dlim) ? e[col + 2 * x + 1] : 0u;
                r[x] = lo | (hi << 16);
            }
        }
    }
    return r;
}

template <int DC, int DO>
struct TriConfig {
    // Rows of X per wavefront: 64 when X fragments (DC/2 regs) plus Out
    // accumulators (DO regs) leave room in the 512-register budget, else 32.
    static constexpr int MW = (DC / 2 + DO <= 192) ? 64 : 32;
    static constexpr int NW = 4;
    static constexpr int BM = MW * NW;
    static constexpr int BN = 64;
    static constexpr int PAD_Y = 16;  // bytes; row stride % 128 == 16 spreads ds_read_b128 rows over banks
    static constexpr int PAD_Z = 64;  // bytes; row stride % 256 == 64 spreads the 4-row transposing reads
    static constexpr int SY = DC * 2 + PAD_Y;
    static constexpr int SZ = DO * 2 + PAD_Z;
    static constexpr int Y_BYTES = BN * SY;
    static constexpr int Z_BYTES = BN * SZ;
    static constexpr int STAGE_BYTES = Y_BYTES + Z_BYTES;
    static constexpr int SMEM_BYTES = 2 * STAGE_BYTES;
};

template <typename T, int DC, int DO>
__global__ __launch_bounds__(256) void tri_xyt_z_kernel(const TriParams p) {
    using Cfg = TriConfig<DC, DO>;
    using M = Mma<T>;
    using V8 = typename M::V8;
    constexpr int MW = Cfg::MW, BM = Cfg::BM, BN = Cfg::BN;
    constexpr int NIB = MW / 32, NBLK = BM / 32;
    constexpr int KC = DC / 16, DB = DO / 32;
    constexpr int SY = Cfg::SY, SZ = Cfg::SZ;
    constexpr int CY = DC / 8, CZ = DO / 8;         // 16-byte chunks per row
    constexpr int NCY = BN * CY / 256, NCZ = BN * CZ / 256;  // chunks per thread per tile
    static_assert(BN * CY % 256 == 0 && BN * CZ % 256 == 0, "tile must split evenly over 256 threads");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, g = lane >> 5;

    // workgroup -> (head, tile): xcd = id % 8 owns heads xcd, xcd+8, ...; within
    // an XCD heads run in sequence, each with its heaviest tile first.
    const int wg = blockIdx.x, xcd = wg & 7, slot = wg >> 3;
    const int hl = slot / p.n_tiles, rank = slot - hl * p.n_tiles;
    const int bh = hl * 8 + xcd;
    if (bh >= p.BH) return;
    const bool upper = p.upper != 0;
    const int tile = upper ? rank : (p.n_tiles - 1 - rank);
    const int b = bh / p.H, h = bh - b * p.H;
    const T *X = static_cast<const T *>(p.x) + b * p.xs_b + h * p.xs_h;
    const T *Y = static_cast<const T *>(p.y) + b * p.ys_b + h * p.ys_h;
    const T *Z = static_cast<const T *>(p.z) + b * p.zs_b + h * p.zs_h;
    T *O = static_cast<T *>(p.out) + b * p.os_b + h * p.os_h;
    const int N = p.N;
    const int i0 = tile * BM;

    // 32-row blocks of this wavefront inside the tile.  With two blocks per
    // wavefront, pair block w with block NBLK-1-w: on the diagonal tile every
    // wavefront then has the same number of unmasked sub-tiles.
    int blk[NIB];
    blk[0] = wave;
    if constexpr (NIB == 2) blk[1] = NBLK - 1 - wave;

    // resident X fragments: B operand of S^T = Y X^T (n = row of X, k = column)
    V8 xf[NIB][KC];
#pragma unroll
    for (int ib = 0; ib < NIB; ++ib) {
        const int row = i0 + blk[ib] * 32 + l32;
        const T *rp = X + (int64_t)row * p.xs_n;
#pragma unroll
        for (int kc = 0; kc < KC; ++kc)
            xf[ib][kc] = __builtin_bit_cast(V8, load8(rp, row < N, kc * 16 + 8 * g, p.dc, p.vec_x != 0));
    }

    f32x16 acc[NIB][DB];
#pragma unroll
    for (int ib = 0; ib < NIB; ++ib)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[ib][db][v] = 0.f;

    // tiles of Y/Z this workgroup visits
    const int jt_begin = upper ? (i0 / BN) : 0;
    const int j_end = upper ? N : (i0 + BM < N ? i0 + BM : N);
    const int jt_end = (j_end + BN - 1) / BN;

    u32x4 ystage[NCY], zstage[NCZ];
    auto fetch = [&](int jt) {
        const int jbase = jt * BN;
#pragma unroll
        for (int u = 0; u < NCY; ++u) {
            const int c = tid + 256 * u, r = c / CY, c8 = c - r * CY;
            const int row = jbase + r;
            ystage[u] = load8(Y + (int64_t)row * p.ys_n, row < N, c8 * 8, p.dc, p.vec_y != 0);
        }
#pragma unroll
        for (int u = 0; u < NCZ; ++u) {
            const int c = tid + 256 * u, r = c / CZ, c8 = c - r * CZ;
            const int row = jbase + r;
            zstage[u] = load8(Z + (int64_t)row * p.zs_n, row < N, c8 * 8, p.dout, p.vec_z != 0);
        }
    };
    auto commit = [&](int buf) {
        unsigned char *yb = smem + buf * Cfg::STAGE_BYTES;
        unsigned char *zb = yb + Cfg::Y_BYTES;
#pragma unroll
        for (int u = 0; u < NCY; ++u) {
            const int c = tid + 256 * u, r = c / CY, c8 = c - r * CY;
            *reinterpret_cast<u32x4 *>(yb + r * SY + c8 * 16) = ystage[u];
        }
#pragma unroll
        for (int u = 0; u < NCZ; ++u) {
            const int c = tid + 256 * u, r = c / CZ, c8 = c - r * CZ;
            *reinterpret_cast<u32x4 *>(zb + r * SZ + c8 * 16) = zstage[u];
        }
    };

    if (jt_begin < jt_end) {
        fetch(jt_begin);
        commit(0);
    }
    __syncthreads();

    // per-lane constant parts of the LDS read addresses
    const int y_lane_off = l32 * SY + g * 16;
    const int z_lane_off = (4 * g + ((lane & 15) >> 2)) * SZ + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;

    int buf = 0;
    for (int jt = jt_begin; jt < jt_end; ++jt) {
        const bool has_next = jt + 1 < jt_end;
        if (has_next) fetch(jt + 1);

        const unsigned char *yb = smem + buf * Cfg::STAGE_BYTES;
        const unsigned char *zb = yb + Cfg::Y_BYTES;
#pragma unroll
        for (int sub = 0; sub < BN / 32; ++sub) {
            const int j0 = jt * BN + sub * 32;
            // 0: fully masked, 1: fully kept, 2: straddles the diagonal
            int st[NIB];
            bool any = false;
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib) {
                const int ib0 = i0 + blk[ib] * 32;
                if (upper)
                    st[ib] = (j0 < ib0) ? 0 : (j0 == ib0 ? 2 : 1);
                else
                    st[ib] = (j0 > ib0) ? 0 : (j0 == ib0 ? 2 : 1);
                any = any || st[ib] != 0;
            }
            if (!any || j0 >= N) continue;

            // S^T[j][i] for the sub-tile
            f32x16 s[NIB];
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib)
#pragma unroll
                for (int v = 0; v < 16; ++v) s[ib][v] = 0.f;
#pragma unroll
            for (int kc = 0; kc < KC; ++kc) {
                const V8 yf = __builtin_bit_cast(
                    V8, *reinterpret_cast<const u32x4 *>(yb + sub * 32 * SY + y_lane_off + kc * 32));
#pragma unroll
                for (int ib = 0; ib < NIB; ++ib) s[ib] = M::mma(yf, xf[ib][kc], s[ib]);
            }

            // mask, round to 16 bit: P fragments (A operand, row = i, k-slot s <-> j = 16t + 8(s/4) + 4g + s%4)
            V8 pf[NIB][2];
#pragma unroll
            for (int ib = 0; ib < NIB; ++ib) {
                if (st[ib] != 1) {
                    const int il = l32;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int jl = 8 * (v / 4) + 4 * g + (v % 4);
                        const bool keep = st[ib] == 2 && (upper ? il <= jl : il >= jl);
                        s[ib][v] = keep ? s[ib][v] : 0.f;
                    }
                }
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int e = 0; e < 8; ++e) pf[ib][t][e] = static_cast<T>(s[ib][8 * t + e]);
            }

            // Out += P Z
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const unsigned char *zp = zb + (sub * 32 + 16 * t) * SZ + z_lane_off + db * 64;
                    typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
                    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(zp));
                    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(zp + 8 * SZ));
                    typedef short s16x8 __attribute__((ext_vector_type(8)));
                    const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    const V8 zf = __builtin_bit_cast(V8, both);
#pragma unroll
                    for (int ib = 0; ib < NIB; ++ib) acc[ib][db] = M::mma(pf[ib][t], zf, acc[ib][db]);
                }
            }
        }

        if (has_next) commit(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    // epilogue: acc[ib][db][v] is Out[row = 8(v/4) + 4g + v%4][col = 32 db + l32] of block ib
#pragma unroll
    for (int ib = 0; ib < NIB; ++ib) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = i0 + blk[ib] * 32 + 8 * (v / 4) + 4 * g + (v % 4);
            if (row < N) {
                T *rp = O + (int64_t)row * p.os_n;
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const int col = db * 32 + l32;
                    if (col < p.dout) rp[col] = static_cast<T>(acc[ib][db][v]);
                }
            }
        }
    }
}

// Launch one instantiation.  Returns hipSuccess or the launch error.
template <typename T, int DC, int DO>
hipError_t launch_tri(TriParams p, hipStream_t stream) {
    using Cfg = TriConfig<DC, DO>;
    if (p.N <= 0 || p.BH <= 0) return hipSuccess;
    p.n_tiles = (p.N + Cfg::BM - 1) / Cfg::BM;
    const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * p.n_tiles;
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    constexpr auto kern = tri_xyt_z_kernel<T, DC, DO>;
    if (hipError_t e = ensure_dynamic_lds<kern>(Cfg::SMEM_BYTES)) return e;
    return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), Cfg::SMEM_BYTES, stream, p);
}

}  // namespace fla

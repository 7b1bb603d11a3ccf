// Chunk states for the chunked evaluation of Out = mask(X Y^T) Z.
//
// With the rows cut into chunks of BM rows (the row tile of the main kernel),
//
//     Out_c = mask(X_c Y_c^T) Z_c  +  X_c . S_c ,    S_c = sum over chunks c' before c (lower mask)
//                                                         or after c (upper mask) of Y_c'^T Z_c'
//
// so everything off the diagonal blocks collapses into a D_c x D_o state per chunk:
// O(N BM D + N D_c D_o) work instead of O(N^2 D).  Two kernels prepare the states:
//
//   chunk_state_kernel : W_c^T = Z_c^T Y_c for every chunk, fp32, [BH][chunks][DO][DC]
//                        (both MFMA operands are column reads of row-major LDS tiles, i.e.
//                        ds_read_b64_tr_b16; the kernel reads Y and Z once and is HBM-bound)
//   chunk_scan_kernel  : exclusive prefix (lower) or suffix (upper) sum over the chunks in fp32,
//                        rounded once to the 16-bit storage type the main kernel multiplies with
//
// The main kernel (fla_tri_fast.h, TriParams::state) then adds X_c . S_c after its diagonal block.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fla_tri_fast.h"

namespace fla {

struct ChunkStateParams {
    const void *y, *z;
    float *w;  // [BH][n_chunks][DO][DC] fp32, padded widths
    int64_t ys_b, ys_h, ys_n;
    int64_t zs_b, zs_h, zs_n;
    int32_t H, N, BH;
    int32_t dc, dout;
    int32_t n_chunks;
    // Feature map on load (fla_feature.h): map_y != 0 replaces every element of Y by phi(element) as
    // the tiles arrive, and writes the mapped rows to `ymap_out` (Y's shape, element strides yo_*) so
    // that the passes after this one read phi(y) instead of mapping again.
    int32_t map_y;
    void *ymap_out;
    int64_t yo_b, yo_h, yo_n;
};

// LDS footprint of the state kernel: at most half of the CU's 160 KiB, so that two workgroups fit
template <int DC, int DO>
struct ChunkStateLds {
    using Cfg = FastConfig<DC, DO>;
    static constexpr int kTiles = Cfg::BM / Cfg::BN;
    static constexpr int kRoundTiles = (kTiles * Cfg::STAGE_BYTES > 80 * 1024 && kTiles % 2 == 0) ? kTiles / 2 : kTiles;
    static constexpr int kBytes = kRoundTiles * Cfg::STAGE_BYTES;
};

template <typename T, int DC, int DO>
__global__ __launch_bounds__(256) void chunk_state_kernel(const ChunkStateParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    using Cfg = FastConfig<DC, DO>;
    using M = Mma<T>;
    using V8 = typename M::V8;
    constexpr int BM = Cfg::BM, BN = Cfg::BN;
    constexpr int RY = Cfg::RY, RZ = Cfg::RZ, CY = Cfg::CY, CZ = Cfg::CZ;
    constexpr int NIY = Cfg::NIY, NIZ = Cfg::NIZ;
    constexpr int STAGE = Cfg::STAGE_BYTES, Y_BYTES = Cfg::Y_BYTES;
    constexpr int NTILE = BM / BN;  // 64-row tiles per chunk
    // tiles resident in LDS at once: the whole chunk when that leaves room for two workgroups
    // per CU (one loads while the other computes), else half of it, in two rounds
    constexpr int RT = ChunkStateLds<DC, DO>::kRoundTiles;
    static_assert(RT <= Cfg::NBUF && NTILE % RT == 0, "a round must fit in LDS and divide the chunk");
    constexpr int EB = DO / 32, DBK = DC / 32;     // 32 x 32 output blocks
    constexpr int NBW = (EB * DBK + 3) / 4;        // blocks per wave (block b goes to wave b % 4)

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5, lam = lane & 15, l32 = lane & 31, beta = (lane >> 4) & 1;

    const int wg = blockIdx.x, xcd = wg & 7, slot = wg >> 3;
    const int hl = slot / p.n_chunks, chunk = slot - hl * p.n_chunks;
    const int bh = hl * 8 + xcd;
    if (bh >= p.BH) return;
    const int b = bh / p.H, h = bh - b * p.H;
    const T *Y = static_cast<const T *>(p.y) + b * p.ys_b + h * p.ys_h;
    const T *Z = static_cast<const T *>(p.z) + b * p.zs_b + h * p.zs_h;
    const int N = p.N, r0 = chunk * BM;
    const int ys2 = (int)p.ys_n * 2, zs2 = (int)p.zs_n * 2;
    const u32x4 ry = make_rsrc(Y, (uint32_t)((N - 1) * ys2 + p.dc * 2));
    const u32x4 rz = make_rsrc(Z, (uint32_t)((N - 1) * zs2 + p.dout * 2));

    // whole chunk -> LDS (rows beyond N and columns beyond the true widths arrive as zeros);
    // same lane -> chunk assignment as the main kernel's tile loads
    constexpr int YSTEP = 4 * (1024 / RY), ZSTEP = 4 * (1024 / RZ);
    constexpr int NYD = Cfg::NYD;
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
    // (the load instruction takes its descriptor, LDS base and row offset in scalar registers;
    // the values are uniform, and said to be so where the compiler loses track of it)
    auto uniform = [](uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); };
    auto uniform4 = [&](const u32x4 &r) {
        u32x4 o = {uniform(r[0]), uniform(r[1]), uniform(r[2]), uniform(r[3])};
        return o;
    };
    auto load_round = [&](auto rr) {
        constexpr int R = decltype(rr)::value;
        const u32x4 ryu = uniform4(ry), rzu = uniform4(rz);
        const uint32_t ldsu = uniform(lds_wave);
        static_for<0, RT>([&](auto tt) {
            constexpr int t = decltype(tt)::value;
            const int row0 = r0 + (R * RT + t) * BN;
            static_for<0, NIY>([&](auto u) {
                constexpr int U = decltype(u)::value;
                dma_16B_per_lane<t * STAGE + U * 4096>(ryu, ldsu, ydma[U % NYD],
                                                       uniform((uint32_t)((row0 + (U - U % NYD) * YSTEP) * ys2)));
            });
            static_for<0, NIZ>([&](auto u) {
                constexpr int U = decltype(u)::value;
                dma_16B_per_lane<t * STAGE + Y_BYTES + U * 4096>(rzu, ldsu, zdma,
                                                                 uniform((uint32_t)((row0 + U * ZSTEP) * zs2)));
            });
        });
        wait_vm<0>();
        __builtin_amdgcn_s_barrier();
        if (p.map_y) {
            // Feature map on load: every thread rewrites its share of the landed Y tiles in place
            // (16 bytes at a time; rows beyond the sequence and chunks beyond the true width arrived
            // as zeros and stay zeros) and stores the mapped values to ymap_out.
            T *YO = static_cast<T *>(p.ymap_out) + b * p.yo_b + h * p.yo_h;
#pragma unroll
            for (int t = 0; t < RT; ++t) {
                unsigned char *tile = smem + t * STAGE;
                const int row0 = r0 + (R * RT + t) * BN;
#pragma unroll
                for (int v = 0; v < BN * CY / 256; ++v) {
                    const int u = tid + 256 * v, r = u / CY, pos = u % CY, c = pos ^ swizzle_y<CY>(r);
                    if (row0 + r < N && c * 8 < p.dc) {
                        u32x4 *ptr = reinterpret_cast<u32x4 *>(tile + r * RY + (pos << 4));
                        const u32x4 m = feature_map8<T>(p.map_y, *ptr);
                        *ptr = m;
                        *reinterpret_cast<u32x4 *>(YO + (int64_t)(row0 + r) * p.yo_n + c * 8) = m;
                    }
                }
            }
            __syncthreads();
        }
    };

    // Column fragment of a row-major tile: rows R0 + {4g..4g+3, 8+4g..8+4g+3}, column 32 cb + l32.
    // Source lane `lam` of a 16-lane group addresses row lam/4, chunk lam%4 of the 16 columns
    // 32 cb + 16 beta .. +15 (plain, unpermuted mapping: destination lane i gets column i).
    auto col_frag = [&](const unsigned char *tile, int rowbytes, int cb, int R0, auto swz) -> V8 {
        const int row_lo = R0 + 4 * g + (lam >> 2), row_hi = row_lo + 8;
        const int chunk16 = 4 * cb + 2 * beta + ((lam & 3) >> 1), sub = 8 * (lam & 1);
        const unsigned char *plo = tile + row_lo * rowbytes + ((chunk16 ^ swz(row_lo)) << 4) + sub;
        const unsigned char *phi = tile + row_hi * rowbytes + ((chunk16 ^ swz(row_hi)) << 4) + sub;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(plo));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(phi));
        return __builtin_bit_cast(V8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    f32x16 acc[NBW];
#pragma unroll
    for (int i = 0; i < NBW; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

    static_for<0, NTILE / RT>([&](auto rr) {
        if constexpr (decltype(rr)::value > 0) __builtin_amdgcn_s_barrier();  // the previous round's tiles are read
        load_round(rr);
#pragma unroll 1
        for (int t = 0; t < RT; ++t) {
            const unsigned char *ytile = smem + t * STAGE, *ztile = ytile + Y_BYTES;
#pragma unroll
            for (int ks = 0; ks < BN / 16; ++ks) {
#pragma unroll
                for (int i = 0; i < NBW; ++i) {
                    const int blk = wave + 4 * i;  // = eb * DBK + dbk
                    if (blk < EB * DBK) {
                        const int eb = blk / DBK, dbk = blk % DBK;
                        const V8 a = col_frag(ztile, RZ, eb, 16 * ks, [](int r) { return swizzle_z<CZ>(r); });
                        const V8 bfr = col_frag(ytile, RY, dbk, 16 * ks, [](int r) { return swizzle_y<CY>(r); });
                        acc[i] = M::mma(a, bfr, acc[i]);
                    }
                }
            }
        }
    });

    // acc[i][v] = W^T[e = 32 eb + 8(v/4) + 4g + v%4][d = 32 dbk + l32]
    float *W = p.w + ((int64_t)bh * p.n_chunks + chunk) * (DO * DC);
#pragma unroll
    for (int i = 0; i < NBW; ++i) {
        const int blk = wave + 4 * i;
        if (blk < EB * DBK) {
            const int eb = blk / DBK, dbk = blk % DBK;
#pragma unroll
            for (int v = 0; v < 16; ++v) W[(32 * eb + 8 * (v / 4) + 4 * g + (v % 4)) * DC + 32 * dbk + l32] = acc[i][v];
        }
    }
#else
    (void)p;
#endif
}

// Exclusive running sum over the chunk axis of w[bh][chunk][E] (fp32), rounded to T.
// reverse == 0: state[c] = sum_{c' < c} w[c'];  reverse != 0: state[c] = sum_{c' > c} w[c'].
// One thread per pair of elements (many sequences have few (b, h) pairs, so parallelism has to
// come from the state elements); the chunk loop runs in batches of 16 (then 4) independent loads
// per thread.
template <typename T>
__global__ __launch_bounds__(256) void chunk_scan_kernel(const float *w, T *state, int n_chunks, int64_t E,
                                                        int64_t total2, int reverse) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef T t2 __attribute__((ext_vector_type(2)));
    const int64_t i2 = (int64_t)blockIdx.x * 256 + threadIdx.x;  // index of a pair of elements within [BH][E]
    if (i2 >= total2) return;
    const int64_t bh = (i2 * 2) / E, e = (i2 * 2) - bh * E;
    const float *wp = w + bh * n_chunks * E + e;
    T *sp = state + bh * n_chunks * E + e;
    const int64_t step = reverse ? -E : E;
    if (reverse) {
        wp += (int64_t)(n_chunks - 1) * E;
        sp += (int64_t)(n_chunks - 1) * E;
    }
    f32x2 run = {0.f, 0.f};
    int k = 0;
    auto batch = [&](auto nn) {
        constexpr int NB = decltype(nn)::value;
        for (; k + NB <= n_chunks; k += NB) {
            f32x2 v[NB];
#pragma unroll
            for (int u = 0; u < NB; ++u) v[u] = *reinterpret_cast<const f32x2 *>(wp + u * step);
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                t2 o;
                o[0] = static_cast<T>(run[0]);
                o[1] = static_cast<T>(run[1]);
                *reinterpret_cast<t2 *>(sp + u * step) = o;
                run += v[u];
            }
            wp += NB * step;
            sp += NB * step;
        }
    };
    batch(std::integral_constant<int, 16>{});
    batch(std::integral_constant<int, 4>{});
    for (; k < n_chunks; ++k) {
        t2 o;
        o[0] = static_cast<T>(run[0]);
        o[1] = static_cast<T>(run[1]);
        *reinterpret_cast<t2 *>(sp) = o;
        run += *reinterpret_cast<const f32x2 *>(wp);
        wp += step;
        sp += step;
    }
}

template <typename T, int DC, int DO>
hipError_t launch_chunk_state(ChunkStateParams p, hipStream_t stream) {
    using Cfg = FastConfig<DC, DO>;
    if constexpr (!Cfg::kSupported) {
        return hipErrorNotSupported;
    } else {
        const int64_t grid = (int64_t)8 * ((p.BH + 7) / 8) * p.n_chunks;
        if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
        constexpr auto kern = chunk_state_kernel<T, DC, DO>;
        constexpr int smem = ChunkStateLds<DC, DO>::kBytes;
        if (hipError_t e = ensure_dynamic_lds<kern>(smem)) return e;
        return launch_kernel<kern>(dim3((unsigned)grid), dim3(256), smem, stream, p);
    }
}

template <typename T>
hipError_t launch_chunk_scan(const float *w, void *state, int64_t BH, int n_chunks, int64_t E, int reverse,
                             hipStream_t stream) {
    const int64_t total2 = BH * E / 2;
    const int64_t grid = (total2 + 255) / 256;
    if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    return launch_kernel<chunk_scan_kernel<T>>(dim3((unsigned)grid), dim3(256), 0, stream, w, static_cast<T *>(state),
                         n_chunks, E, total2, reverse);
}

}  // namespace fla

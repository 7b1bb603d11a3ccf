// The normaliser of causal linear attention, fused into four memory-bound kernels:
//
//     n_i   = q_i . (k_0 + ... + k_i) + eps          out_i = O_i / n_i
//
// (the recipe the reference leaves to the caller in PyTorch, README.md:27-30: a cumsum over k,
// an elementwise product with q, a row sum, an add and a division) and its backward.  With
// g = d(out), the unnormalised product's gradient and the normaliser's own terms are
//
//     dO_i = g_i / n_i        dn_i = -(g_i . out_i) / n_i
//     dq_i += dn_i (k_0 + ... + k_i)        dk_j += dn_j q_j + ... + dn_{N-1} q_{N-1}
//
// Everything is a running sum along the sequence, so a (batch, head) slice is cut into chunks
// of R rows: one kernel writes per-chunk column sums, a tiny kernel turns them into exclusive
// prefix (suffix) sums over the chunks, and the consumer scans its own rows starting from its
// chunk's entry.  Inside a chunk every group of LPR lanes owns a segment of 16 consecutive rows
// (8 columns per lane, kept packed in registers), segment totals are exchanged through LDS, and
// each row is visited once more with the right offset.  All loads of a workgroup are issued
// before the first use.  Arithmetic is fp32 throughout; inputs and outputs are the 16-bit
// storage type.  VEC = true instantiations assume every operand qualifies for 16-byte accesses.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fla_feature.h"
#include "fla_tri_kernel.h"

namespace fla {

constexpr int kNormSegRows = 16;  // rows per segment (kept packed in registers)

struct NormParams {
    const void *q, *k;       // (B, H, N, dqk)
    const void *a;           // fwd: unnormalised O; bwd-pre: grad of the normalised output; (B, H, N, dv)
    const void *b;           // bwd-pre: the normalised output saved by forward; (B, H, N, dv)
    void *out;               // fwd: normalised output; bwd-pre: dO = g / n (contiguous); (B, H, N, dv)
    void *dq, *dk;           // bwd-post: gradients, updated in place; (B, H, N, dqk)
    float *denom;            // n, fp32, contiguous (B H, N)
    float *dn;               // bwd: dn, fp32, contiguous (B H, N)
    float *ksum, *wsum;      // per-chunk column sums of k and of dn q: fp32 [B H][chunks][DP]
    int64_t qs_b, qs_h, qs_n, ks_b, ks_h, ks_n;
    int64_t as_b, as_h, as_n, bs_b, bs_h, bs_n, os_b, os_h, os_n;
    int64_t dqs_b, dqs_h, dqs_n, dks_b, dks_h, dks_n;
    int32_t H, N, BH, dqk, dv, n_chunks;
    int32_t vec_q, vec_k, vec_a, vec_b, vec_out, vec_dq, vec_dk;
    float eps;
    // bwd-post with a feature map (fla_feature.h): q and k hold y = phi(x), and the finished
    // gradients are multiplied by phi'(x) computed from y -- they leave as gradients with respect
    // to x.  0: none.
    int32_t fmap;
    int32_t only_dk;  // bwd-post: only the dk half (dq is complete)
};

template <typename T>
__device__ __forceinline__ void unpack8(u32x4 w, float (&f)[8]) {
    typedef T v8 __attribute__((ext_vector_type(8)));
    const v8 x = __builtin_bit_cast(v8, w);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = static_cast<float>(x[e]);
}
template <typename T>
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
    typedef T v8 __attribute__((ext_vector_type(8)));
    v8 x;
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = static_cast<T>(f[e]);
    return __builtin_bit_cast(u32x4, x);
}
template <typename T>
__device__ __forceinline__ void store8(T *row, int col, int dlim, bool vec, u32x4 w) {
    if (col >= dlim) return;
    if (vec) {
        *reinterpret_cast<u32x4 *>(row + col) = w;
    } else {
        unsigned short *e = reinterpret_cast<unsigned short *>(row);
#pragma unroll
        for (int x = 0; x < 8; ++x)
            if (col + x < dlim) e[col + x] = (unsigned short)(w[x >> 1] >> (16 * (x & 1)));
    }
}
// sum over the LPR lanes that share a row (LPR a power of two, lanes contiguous)
template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
    for (int m = 1; m < LPR; m <<= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// Geometry shared by the kernels: 256 threads, LPR lanes per row, 64 / LPR row slots per wave,
// 4 waves -> NSEG segments of kNormSegRows rows each.
template <int LPR>
struct NormGeom {
    static constexpr int RPS = 64 / LPR;
    static constexpr int NSEG = 4 * RPS;
    static constexpr int R = NSEG * kNormSegRows;  // rows per chunk
    static constexpr int DP = LPR * 8;             // padded width
};

// ---- per-chunk column sums: ksum = sum k_r, and (WITH_W) wsum = sum dn_r q_r
template <typename T, int LPR, bool VEC, bool WITH_W>
__global__ __launch_bounds__(256) void norm_chunk_sums_kernel(const NormParams p) {
    using G = NormGeom<LPR>;
    __shared__ float red[(WITH_W ? 2 : 1) * G::NSEG * G::DP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane % LPR, seg = wave * G::RPS + lane / LPR;
    const int chunk = blockIdx.x, bh = blockIdx.y;
    const int b = bh / p.H, h = bh - b * p.H;
    const T *K = static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h;
    const T *Q = static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h;
    const int row0 = chunk * G::R + seg * kNormSegRows, col = 8 * li;
    u32x4 kr[kNormSegRows], qr[WITH_W ? kNormSegRows : 1];
    float dn[WITH_W ? kNormSegRows : 1];
#pragma unroll
    for (int r = 0; r < kNormSegRows; ++r) {
        const int row = row0 + r;
        const bool ok = row < p.N;
        kr[r] = load8(K + (int64_t)row * p.ks_n, ok, col, p.dqk, VEC || p.vec_k != 0);
        if constexpr (WITH_W) {
            qr[r] = load8(Q + (int64_t)row * p.qs_n, ok, col, p.dqk, VEC || p.vec_q != 0);
            dn[r] = ok ? p.dn[(int64_t)bh * p.N + row] : 0.f;
        }
    }
    float sk[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, sw[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < kNormSegRows; ++r) {
        float kf[8];
        unpack8<T>(kr[r], kf);
#pragma unroll
        for (int e = 0; e < 8; ++e) sk[e] += kf[e];
        if constexpr (WITH_W) {
            float qf[8];
            unpack8<T>(qr[r], qf);
#pragma unroll
            for (int e = 0; e < 8; ++e) sw[e] += dn[r] * qf[e];
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        red[seg * G::DP + col + e] = sk[e];
        if constexpr (WITH_W) red[(G::NSEG + seg) * G::DP + col + e] = sw[e];
    }
    __syncthreads();
    for (int c = tid; c < (WITH_W ? 2 : 1) * G::DP; c += 256) {
        const int which = c / G::DP, cc = c - which * G::DP;
        float t = 0.f;
#pragma unroll
        for (int s = 0; s < G::NSEG; ++s) t += red[(which * G::NSEG + s) * G::DP + cc];
        float *dst = which ? p.wsum : p.ksum;
        dst[((int64_t)bh * p.n_chunks + chunk) * G::DP + cc] = t;
    }
}

// ---- chunk sums -> exclusive prefix sums over the chunks (ksum) and exclusive suffix sums
// (wsum, when given), in place.  One thread per (batch-head, column).  (A template only so that the
// definition may sit in a header that several translation units include.)
template <int kUnused = 0>
__global__ __launch_bounds__(256) void norm_scan_kernel(float *ksum, float *wsum, int BH, int chunks, int DP) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= (int64_t)BH * DP) return;
    const int64_t bh = t / DP, c0 = t - bh * DP;
    float *ks = ksum + bh * chunks * DP + c0;
    float run = 0.f;
    for (int c = 0; c < chunks; ++c) {
        const float v = ks[(int64_t)c * DP];
        ks[(int64_t)c * DP] = run;
        run += v;
    }
    if (wsum) {
        float *ws = wsum + bh * chunks * DP + c0;
        run = 0.f;
        for (int c = chunks - 1; c >= 0; --c) {
            const float v = ws[(int64_t)c * DP];
            ws[(int64_t)c * DP] = run;
            run += v;
        }
    }
}

// ---- forward: n_i = q_i . cumsum(k)_i + eps, out_i = a_i / n_i (a = unnormalised O; may alias out)
template <typename T, int LPR, bool VEC>
__global__ __launch_bounds__(256, 2) void norm_fwd_kernel(const NormParams p) {
    using G = NormGeom<LPR>;
    __shared__ float tot[G::NSEG * G::DP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane % LPR, seg = wave * G::RPS + lane / LPR;
    const int chunk = blockIdx.x, bh = blockIdx.y;
    const int b = bh / p.H, h = bh - b * p.H;
    const T *K = static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h;
    const T *Q = static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h;
    const T *A = static_cast<const T *>(p.a) + b * p.as_b + h * p.as_h;
    T *O = static_cast<T *>(p.out) + b * p.os_b + h * p.os_h;
    const int row0 = chunk * G::R + seg * kNormSegRows, col = 8 * li;

    // this segment's rows of k and q, packed; all requested before anything is used
    u32x4 kr[kNormSegRows], qr[kNormSegRows];
#pragma unroll
    for (int r = 0; r < kNormSegRows; ++r)
        kr[r] = load8(K + (int64_t)(row0 + r) * p.ks_n, row0 + r < p.N, col, p.dqk, VEC || p.vec_k != 0);
#pragma unroll
    for (int r = 0; r < kNormSegRows; ++r)
        qr[r] = load8(Q + (int64_t)(row0 + r) * p.qs_n, row0 + r < p.N, col, p.dqk, VEC || p.vec_q != 0);
    float run[8];
    if (chunk > 0) {
        const float *src = p.ksum + ((int64_t)bh * p.n_chunks + chunk) * G::DP + col;
#pragma unroll
        for (int e = 0; e < 8; ++e) run[e] = src[e];
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) run[e] = 0.f;
    }
    {
        float t[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < kNormSegRows; ++r) {
            float kf[8];
            unpack8<T>(kr[r], kf);
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] += kf[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) tot[seg * G::DP + col + e] = t[e];
    }
    __syncthreads();
    for (int s = 0; s < seg; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) run[e] += tot[s * G::DP + col + e];

    // normalisers of the segment's rows, then the division row by row
    float inv[kNormSegRows];
#pragma unroll
    for (int r = 0; r < kNormSegRows; ++r) {
        float kf[8], qf[8];
        unpack8<T>(kr[r], kf);
        unpack8<T>(qr[r], qf);
        float part = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            run[e] += kf[e];
            part += qf[e] * run[e];
        }
        const float n = row_sum<LPR>(part) + p.eps;
        inv[r] = 1.0f / n;
        if (li == 0 && row0 + r < p.N) p.denom[(int64_t)bh * p.N + row0 + r] = n;
    }
    if (col >= p.dv) return;
    constexpr int HALF = kNormSegRows / 2;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        u32x4 ar[HALF];
#pragma unroll
        for (int r = 0; r < HALF; ++r) {
            const int row = row0 + half * HALF + r;
            ar[r] = load8(A + (int64_t)row * p.as_n, row < p.N, col, p.dv, VEC || p.vec_a != 0);
        }
#pragma unroll
        for (int r = 0; r < HALF; ++r) {
            const int row = row0 + half * HALF + r;
            if (row < p.N) {
                float af[8];
                unpack8<T>(ar[r], af);
#pragma unroll
                for (int e = 0; e < 8; ++e) af[e] *= inv[half * HALF + r];
                store8<T>(O + (int64_t)row * p.os_n, col, p.dv, VEC || p.vec_out != 0, pack8<T>(af));
            }
        }
    }
}

// ---- backward, before the main gradient kernels: dO = g / n (contiguous), dn = -(g . out) / n
template <typename T, int LPR, bool VEC>
__global__ __launch_bounds__(256) void norm_bwd_pre_kernel(const NormParams p) {
    using G = NormGeom<LPR>;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane % LPR, slot = wave * G::RPS + lane / LPR;
    const int bh = blockIdx.y;
    const int b = bh / p.H, h = bh - b * p.H;
    const T *Gr = static_cast<const T *>(p.a) + b * p.as_b + h * p.as_h;
    const T *Ou = static_cast<const T *>(p.b) + b * p.bs_b + h * p.bs_h;
    T *dO = static_cast<T *>(p.out) + b * p.os_b + h * p.os_h;
    const int col = 8 * li;
#pragma unroll 4
    for (int r = 0; r < kNormSegRows; ++r) {
        const int row = (blockIdx.x * kNormSegRows + r) * G::NSEG + slot;  // consecutive rows across the workgroup
        const bool ok = row < p.N;
        float gf[8], of[8];
        unpack8<T>(load8(Gr + (int64_t)row * p.as_n, ok, col, p.dv, VEC || p.vec_a != 0), gf);
        unpack8<T>(load8(Ou + (int64_t)row * p.bs_n, ok, col, p.dv, VEC || p.vec_b != 0), of);
        float part = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) part += gf[e] * of[e];
        const float dot = row_sum<LPR>(part);
        if (ok) {
            const float inv = 1.0f / p.denom[(int64_t)bh * p.N + row];
#pragma unroll
            for (int e = 0; e < 8; ++e) gf[e] *= inv;
            store8<T>(dO + (int64_t)row * p.os_n, col, p.dv, VEC || p.vec_out != 0, pack8<T>(gf));
            if (li == 0) p.dn[(int64_t)bh * p.N + row] = -dot * inv;
        }
    }
}

// ---- backward, after the main gradient kernels.  blockIdx.z = 0: dq_i += dn_i cumsum(k)_i;
// blockIdx.z = 1: dk_j += revcumsum(dn q)_j.  The two halves are independent.
template <typename T, int LPR, bool VEC>
__global__ __launch_bounds__(256, 2) void norm_bwd_post_kernel(const NormParams p) {
    using G = NormGeom<LPR>;
    __shared__ float tot[G::NSEG * G::DP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane % LPR, seg = wave * G::RPS + lane / LPR;
    const int chunk = blockIdx.x, bh = blockIdx.y;
    const bool part_dk = blockIdx.z != 0 || p.only_dk;
    const int b = bh / p.H, h = bh - b * p.H;
    // the scanned operand (k for dq, q for dk) and the gradient that is updated
    const T *S = part_dk ? static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h
                         : static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h;
    const int64_t ss_n = part_dk ? p.qs_n : p.ks_n;
    const bool vec_s = VEC || (part_dk ? p.vec_q : p.vec_k) != 0;
    T *D = part_dk ? static_cast<T *>(p.dk) + b * p.dks_b + h * p.dks_h
                   : static_cast<T *>(p.dq) + b * p.dqs_b + h * p.dqs_h;
    const int64_t ds_n = part_dk ? p.dks_n : p.dqs_n;
    const bool vec_d = VEC || (part_dk ? p.vec_dk : p.vec_dq) != 0;
    const int row0 = chunk * G::R + seg * kNormSegRows, col = 8 * li;

    u32x4 sr[kNormSegRows], dr[kNormSegRows];
    float dn[kNormSegRows];
#pragma unroll
    for (int r = 0; r < kNormSegRows; ++r) {
        const int row = row0 + r;
        sr[r] = load8(S + (int64_t)row * ss_n, row < p.N, col, p.dqk, vec_s);
        dn[r] = row < p.N ? p.dn[(int64_t)bh * p.N + row] : 0.f;
    }
#pragma unroll
    for (int r = 0; r < kNormSegRows; ++r)
        dr[r] = load8(D + (int64_t)(row0 + r) * ds_n, row0 + r < p.N, col, p.dqk, vec_d);
    // with a feature map: the rows of y = phi(x) that belong to the gradient being finished
    // (q for dq, k for dk), for the slope
    u32x4 yr[kNormSegRows];
    if (p.fmap) {
        const T *Yv = part_dk ? static_cast<const T *>(p.k) + b * p.ks_b + h * p.ks_h
                              : static_cast<const T *>(p.q) + b * p.qs_b + h * p.qs_h;
        const int64_t ys_n = part_dk ? p.ks_n : p.qs_n;
        const bool vec_y = VEC || (part_dk ? p.vec_k : p.vec_q) != 0;
#pragma unroll
        for (int r = 0; r < kNormSegRows; ++r)
            yr[r] = load8(Yv + (int64_t)(row0 + r) * ys_n, row0 + r < p.N, col, p.dqk, vec_y);
    }
    // running sum at the entry of this chunk: chunks before it (k) or after it (dn q)
    float run[8];
    {
        const float *src = (part_dk ? p.wsum : p.ksum) + ((int64_t)bh * p.n_chunks + chunk) * G::DP + col;
        const bool have = p.n_chunks > 1;
#pragma unroll
        for (int e = 0; e < 8; ++e) run[e] = have ? src[e] : 0.f;
    }
    {
        float t[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < kNormSegRows; ++r) {
            float sf[8];
            unpack8<T>(sr[r], sf);
            const float w = part_dk ? dn[r] : 1.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] += w * sf[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) tot[seg * G::DP + col + e] = t[e];
    }
    __syncthreads();
    if (part_dk) {
        for (int s = seg + 1; s < G::NSEG; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) run[e] += tot[s * G::DP + col + e];
    } else {
        for (int s = 0; s < seg; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) run[e] += tot[s * G::DP + col + e];
    }
    if (col >= p.dqk) return;
    // inclusive scan over the segment's rows: ascending for dq, descending for dk
#pragma unroll
    for (int i = 0; i < kNormSegRows; ++i) {
        // register arrays are indexed by compile-time constants only: both candidates, then select
        float sf[8], g[8];
        unpack8<T>(part_dk ? sr[kNormSegRows - 1 - i] : sr[i], sf);
        unpack8<T>(part_dk ? dr[kNormSegRows - 1 - i] : dr[i], g);
        const float dnr = part_dk ? dn[kNormSegRows - 1 - i] : dn[i];
        const int row = row0 + (part_dk ? kNormSegRows - 1 - i : i);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            run[e] += (part_dk ? dnr : 1.0f) * sf[e];
            g[e] += (part_dk ? 1.0f : dnr) * run[e];
        }
        if (p.fmap) {
            float yf[8];
            unpack8<T>(part_dk ? yr[kNormSegRows - 1 - i] : yr[i], yf);
#pragma unroll
            for (int e = 0; e < 8; ++e) g[e] *= feature_slope_from_value(p.fmap, yf[e]);
        }
        if (row < p.N) store8<T>(D + (int64_t)row * ds_n, col, p.dqk, vec_d, pack8<T>(g));
    }
}

// lanes per row for a width: the smallest of 4, 8, 16, 32 with 8 LPR >= width
inline int norm_lanes_per_row(int width) { return width <= 32 ? 4 : width <= 64 ? 8 : width <= 128 ? 16 : 32; }
inline int norm_chunk_rows(int lpr) { return 4 * (64 / lpr) * kNormSegRows; }

inline hipError_t launch_norm_scan(const NormParams &p, int dp, bool with_w, hipStream_t s) {
    const int64_t threads = (int64_t)p.BH * dp;
    return launch_kernel<norm_scan_kernel<0>>(dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, p.ksum,
                         with_w ? p.wsum : nullptr, p.BH, p.n_chunks, dp);
}

// which: 0 forward, 1 backward-pre, 2 backward-post
template <typename T, int LPR, bool VEC>
hipError_t launch_norm_lpr(int which, const NormParams &p, hipStream_t s) {
    const dim3 grid((unsigned)p.n_chunks, (unsigned)p.BH);
    // every launch is checked on its own: nothing further is enqueued after a failed one
    if (which == 0) {
        if (p.n_chunks > 1) {
            if (hipError_t e = launch_kernel<norm_chunk_sums_kernel<T, LPR, VEC, false>>(grid, dim3(256), 0, s, p)) return e;
            if (hipError_t e = launch_norm_scan(p, LPR * 8, false, s)) return e;
        }
        return launch_kernel<norm_fwd_kernel<T, LPR, VEC>>(grid, dim3(256), 0, s, p);
    }
    if (which == 1) return launch_kernel<norm_bwd_pre_kernel<T, LPR, VEC>>(grid, dim3(256), 0, s, p);
    if (p.n_chunks > 1) {
        if (hipError_t e = launch_kernel<norm_chunk_sums_kernel<T, LPR, VEC, true>>(grid, dim3(256), 0, s, p)) return e;
        if (hipError_t e = launch_norm_scan(p, LPR * 8, true, s)) return e;
    }
    return launch_kernel<norm_bwd_post_kernel<T, LPR, VEC>>(dim3(grid.x, grid.y, p.only_dk ? 1 : 2), dim3(256), 0, s, p);
}

// lpr from norm_lanes_per_row; vec: every operand of this call qualifies for 16-byte accesses
template <typename T>
hipError_t launch_norm(int which, int lpr, bool vec, const NormParams &p, hipStream_t s) {
#define FLA_NORM_CASE(L) \
    case L: return vec ? launch_norm_lpr<T, L, true>(which, p, s) : launch_norm_lpr<T, L, false>(which, p, s);
    switch (lpr) {
        FLA_NORM_CASE(4)
        FLA_NORM_CASE(8)
        FLA_NORM_CASE(16)
        FLA_NORM_CASE(32)
        default: return hipErrorInvalidValue;
    }
#undef FLA_NORM_CASE
}

}  // namespace fla

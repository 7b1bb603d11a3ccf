// C ABI of libfla_gfx950.so (declared in include/fla.h): argument checks,
// mapping of forward / gradients onto the one masked-product kernel, launch.
#include "fla.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "fla_dispatch.h"
#include "fla_norm.h"

// Scratch of fla_linear_attn_chunked_fwd_static: one copy per GPU, at its own address on each.
// Host code never uses the array's name as an address; it asks the runtime for the device
// address once per device (static_scratch below) and passes that pointer on.  (No `used`
// attribute: it would pin the device symbol to local binding, where the runtime's lookup by
// name cannot find it; the reference from host code below is what keeps the array and makes
// the compiler give it global binding.)
static __device__ __align__(256) unsigned char scratch[FLA_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch(void **out) {
#if defined(FLA_TRACE_LAUNCHES)
    *out = reinterpret_cast<void *>((uintptr_t)0x700000000000ull);  // (no device: a made-up, aligned address)
    return FLA_OK;
#endif
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return FLA_ERR_LAUNCH;
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return FLA_ERR_LAUNCH;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return FLA_OK;
}

using fla::TriParams;
typedef hipError_t (*launch_fn)(const TriParams &, hipStream_t);

int pad_index(int64_t d) { return d <= 32 ? 0 : d <= 64 ? 1 : d <= 128 ? 2 : 3; }

launch_fn lookup(int dtype, int64_t dc, int64_t dout) {
#define FLA_ENTRY(c, o) {fla::FLA_LAUNCH_NAME(0, c, o), fla::FLA_LAUNCH_NAME(1, c, o)},
    static const launch_fn table[16][2] = {FLA_FOR_EACH_DIM_PAIR(FLA_ENTRY)};
#undef FLA_ENTRY
    return table[pad_index(dc) * 4 + pad_index(dout)][dtype];
}

typedef hipError_t (*state_fn)(const fla::ChunkStateParams &, hipStream_t);

state_fn lookup_state(int dtype, int64_t dc, int64_t dout) {
#define FLA_ENTRY(c, o) {fla::FLA_STATE_NAME(0, c, o), fla::FLA_STATE_NAME(1, c, o)},
    static const state_fn table[16][2] = {FLA_FOR_EACH_DIM_PAIR(FLA_ENTRY)};
#undef FLA_ENTRY
    return table[pad_index(dc) * 4 + pad_index(dout)][dtype];
}

// rows per chunk of the chunked evaluation for this pair of widths (0: none available)
int chunk_rows(int64_t dc, int64_t dout) {
#define FLA_ENTRY(c, o) fla::fla_chunk_rows_c##c##_o##o,
    static int (*const table[16])() = {FLA_FOR_EACH_DIM_PAIR(FLA_ENTRY)};
#undef FLA_ENTRY
    return table[pad_index(dc) * 4 + pad_index(dout)]();
}

int64_t padded(int64_t d) { return d <= 32 ? 32 : d <= 64 ? 64 : d <= 128 ? 128 : 256; }

int64_t next_pow2(int64_t x) {
    int64_t p = 1;
    while (p < x) p <<= 1;
    return p;
}

struct View {
    const void *ptr;
    const int64_t *strides;
};

int check_view(const View &t) {
    if (!t.ptr) return FLA_ERR_NULL_POINTER;
    if (!t.strides) return FLA_ERR_STRIDE;
    if (t.strides[3] != 1) return FLA_ERR_STRIDE;
    if (t.strides[0] < 0 || t.strides[1] < 0 || t.strides[2] < 0) return FLA_ERR_STRIDE;
    return FLA_OK;
}

// 16-byte vector loads are legal when every row starts 16-byte aligned and the
// width is a whole number of 8-element chunks.
int vec_ok(const View &t, int64_t width) {
    return width % 8 == 0 && reinterpret_cast<uintptr_t>(t.ptr) % 16 == 0 && t.strides[0] % 8 == 0 &&
           t.strides[1] % 8 == 0 && t.strides[2] % 8 == 0;
}

// The kernels read tiles of the inputs while other workgroups already write results: an output
// that shares memory with an input (or with another output) would be read half-updated.  The
// test is on the byte ranges [first element, one past the last addressed element).
struct Span {
    uintptr_t lo, hi;
};

Span span_of(const View &t, int64_t B, int64_t H, int64_t N, int64_t width) {
    if (B <= 0 || H <= 0 || N <= 0 || !t.ptr || !t.strides) return {0, 0};
    const int64_t last = (B - 1) * t.strides[0] + (H - 1) * t.strides[1] + (N - 1) * t.strides[2] + width;
    const uintptr_t lo = reinterpret_cast<uintptr_t>(t.ptr);
    return {lo, lo + (uintptr_t)last * 2};
}

bool overlap(const Span &a, const Span &b) { return a.lo < b.hi && b.lo < a.hi; }

int check_alias(const Span *ins, int n_in, const Span *outs, int n_out) {
    for (int o = 0; o < n_out; ++o) {
        for (int i = 0; i < n_in; ++i)
            if (overlap(outs[o], ins[i])) return FLA_ERR_ALIAS;
        for (int o2 = o + 1; o2 < n_out; ++o2)
            if (overlap(outs[o], outs[o2])) return FLA_ERR_ALIAS;
    }
    return FLA_OK;
}

int check_common(int64_t B, int64_t H, int64_t N, int dtype) {
    if (dtype != FLA_DTYPE_BF16 && dtype != FLA_DTYPE_F16) return FLA_ERR_DTYPE;
    if (B < 0 || H < 0 || N < 0) return FLA_ERR_SHAPE;
    if (N > (int64_t)1 << 30) return FLA_ERR_SHAPE;
    if (H > 0 && B > ((int64_t)1 << 30) / H) return FLA_ERR_SHAPE;
    return FLA_OK;
}

// forward-shaped call: two operands of width dc and one of width dout in, one of width dout out
int check_alias_fwd(const View &x, const View &y, const View &z, const View &out, int64_t B, int64_t H, int64_t N,
                    int64_t dc, int64_t dout) {
    const Span ins[] = {span_of(x, B, H, N, dc), span_of(y, B, H, N, dc), span_of(z, B, H, N, dout)};
    const Span outs[] = {span_of(out, B, H, N, dout)};
    return check_alias(ins, 3, outs, 1);
}

// backward-shaped call: go, v (and the forward's output `o`, when given) of width dv, q, k of width
// dqk in; dq, dk of width dqk and dv of width dv out
int check_alias_bwd(const View &go, const View &q, const View &k, const View &v, const View *o, const View &dq,
                    const View &dk, const View &dvv, int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv) {
    const Span ins[] = {span_of(go, B, H, N, dv), span_of(q, B, H, N, dqk), span_of(k, B, H, N, dqk),
                        span_of(v, B, H, N, dv), o ? span_of(*o, B, H, N, dv) : Span{0, 0}};
    const Span outs[] = {span_of(dq, B, H, N, dqk), span_of(dk, B, H, N, dqk), span_of(dvv, B, H, N, dv)};
    return check_alias(ins, 5, outs, 3);
}

TriParams make_params(const View &x, const View &y, const View &z, const View &out, int64_t B, int64_t H, int64_t N,
                      int64_t dc, int64_t dout, int upper) {
    TriParams p;
    p.x = x.ptr, p.y = y.ptr, p.z = z.ptr, p.out = const_cast<void *>(out.ptr);
    p.xs_b = x.strides[0], p.xs_h = x.strides[1], p.xs_n = x.strides[2];
    p.ys_b = y.strides[0], p.ys_h = y.strides[1], p.ys_n = y.strides[2];
    p.zs_b = z.strides[0], p.zs_h = z.strides[1], p.zs_n = z.strides[2];
    p.os_b = out.strides[0], p.os_h = out.strides[1], p.os_n = out.strides[2];
    p.H = (int32_t)H, p.N = (int32_t)N, p.BH = (int32_t)(B * H);
    p.dc = (int32_t)dc, p.dout = (int32_t)dout;
    p.upper = upper ? 1 : 0;
    p.n_tiles = 0;
    p.single = 0;
    p.state = nullptr;
    p.state_transposed = 0;
    p.denom = nullptr;
    p.eps = 0.f;
    p.poly[0] = p.poly[1] = p.poly[2] = 0.f;
    p.poly_on = 0;
    p.map_x = p.map_out = 0;
    p.xmap_out = nullptr, p.omap = nullptr;
    p.xo_b = p.xo_h = p.xo_n = 0;
    p.ms_b = p.ms_h = p.ms_n = 0;
    p.vec_x = vec_ok(x, dc), p.vec_y = vec_ok(y, dc), p.vec_z = vec_ok(z, dout), p.vec_out = vec_ok(out, dout);
    return p;
}

typedef hipError_t (*batch_fn)(const fla::TriBatch &, int, hipStream_t);

batch_fn lookup_batch(int dtype, int64_t d) {
    static const batch_fn table[4][2] = {{fla::FLA_BATCH_NAME(0, 32), fla::FLA_BATCH_NAME(1, 32)},
                                         {fla::FLA_BATCH_NAME(0, 64), fla::FLA_BATCH_NAME(1, 64)},
                                         {fla::FLA_BATCH_NAME(0, 128), fla::FLA_BATCH_NAME(1, 128)},
                                         {fla::FLA_BATCH_NAME(0, 256), fla::FLA_BATCH_NAME(1, 256)}};
    return table[pad_index(d)][dtype];
}

batch_fn lookup_chunked_batch(int dtype, int64_t d) {
    static const batch_fn table[4][2] = {{fla::FLA_CBATCH_NAME(0, 32), fla::FLA_CBATCH_NAME(1, 32)},
                                         {fla::FLA_CBATCH_NAME(0, 64), fla::FLA_CBATCH_NAME(1, 64)},
                                         {fla::FLA_CBATCH_NAME(0, 128), fla::FLA_CBATCH_NAME(1, 128)},
                                         {fla::FLA_CBATCH_NAME(0, 256), fla::FLA_CBATCH_NAME(1, 256)}};
    return table[pad_index(d)][dtype];
}

// Out = mask(X Y^T) Z; all arguments already validated.
int run_tri(const View &x, const View &y, const View &z, const View &out, int64_t B, int64_t H, int64_t N,
            int64_t dc, int64_t dout, int upper, int dtype, void *stream) {
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    // Output wider than 128 columns with a narrow (<= 64) or a 256-wide contraction: run the two
    // 128-column halves of Z / Out as separate launches.  The 64-rows-per-wave kernels that
    // this selects beat the single 256-wide launch (which needs the 32-row layout, or the
    // generic kernel for 256 x 256) although S is formed twice; results are bit-identical
    // because every output column is an independent sum.
    if (dout > 128 && (dc <= 64 || dc > 128)) {
        const View z_hi{static_cast<const char *>(z.ptr) + 128 * 2, z.strides};
        const View out_hi{static_cast<const char *>(out.ptr) + 128 * 2, out.strides};
        if (int rc = run_tri(x, y, z, out, B, H, N, dc, 128, upper, dtype, stream)) return rc;
        return run_tri(x, y, z_hi, out_hi, B, H, N, dc, dout - 128, upper, dtype, stream);
    }
    const TriParams p = make_params(x, y, z, out, B, H, N, dc, dout, upper);
    launch_fn fn = lookup(dtype, dc, dout);
    if (!fn) return FLA_ERR_UNSUPPORTED;
    return fn(p, static_cast<hipStream_t>(stream)) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
}

// bytes of workspace the chunked evaluation of one product needs: fp32 chunk states plus
// their 16-bit running sums, [BH][chunks][DO][DC] each with padded widths
int64_t chunked_bytes(int64_t B, int64_t H, int64_t N, int64_t dc, int64_t dout) {
    if (dout > 128 && (dc <= 64 || dc > 128)) dout = 128;  // evaluated as two 128-column halves
    const int rows = chunk_rows(dc, dout);
    if (rows == 0 || N <= rows) return 0;
    const int64_t chunks = (N + rows - 1) / rows;
    return B * H * chunks * padded(dc) * padded(dout) * 6;
}

// ---- element-wise feature passes, for the shapes and layouts the kernels' own map-on-load does
// not cover: mode 1 writes dst = phi(src); mode 2 multiplies dst in place by phi'(x) computed from
// src = phi(x); mode 3 adds src to dst in place (fp32 sum, one rounding).  Any strides; eight elements per thread where both tensors allow 16-byte accesses.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void feature_pass_kernel(int mode, int fmap, const T *src, int64_t ss_b, int64_t ss_h,
                                                           int64_t ss_n, T *dst, int64_t ds_b, int64_t ds_h,
                                                           int64_t ds_n, int H, int64_t N, int D, int64_t total) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    constexpr int E = VEC ? 8 : 1;
    const int per_row = D / E;
    const int64_t row = t / per_row;
    const int col = (int)(t - row * per_row) * E;
    const int64_t bh = row / N, n = row - bh * N;
    const int64_t b = bh / H, h = bh - b * H;
    const T *sp = src + b * ss_b + h * ss_h + n * ss_n + col;
    T *dp = dst + b * ds_b + h * ds_h + n * ds_n + col;
    if constexpr (VEC) {
        typedef T v8 __attribute__((ext_vector_type(8)));
        v8 s = *reinterpret_cast<const v8 *>(sp), d;
        if (mode != 1) d = *reinterpret_cast<const v8 *>(dp);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = static_cast<float>(s[e]);
            d[e] = static_cast<T>(mode == 1   ? fla::feature_value(fmap, x)
                                  : mode == 2 ? static_cast<float>(d[e]) * fla::feature_slope_from_value(fmap, x)
                                              : static_cast<float>(d[e]) + x);
        }
        *reinterpret_cast<v8 *>(dp) = d;
    } else {
        const float x = static_cast<float>(*sp);
        *dp = static_cast<T>(mode == 1   ? fla::feature_value(fmap, x)
                             : mode == 2 ? static_cast<float>(*dp) * fla::feature_slope_from_value(fmap, x)
                                         : static_cast<float>(*dp) + x);
    }
}

int launch_feature_pass(int mode, int fmap, const View &src, const View &dst, int64_t B, int64_t H, int64_t N,
                        int64_t D, int dtype, void *stream) {
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    const bool vec = vec_ok(src, D) && vec_ok(dst, D);
    const int64_t total = B * H * N * (vec ? D / 8 : D);
    const int64_t grid = (total + 255) / 256;
    if (grid > 0x7fffffffLL) return FLA_ERR_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
#define FLA_FEATURE_PASS(T, V)                                                                                      \
    fla::launch_kernel<feature_pass_kernel<T, V>>(dim3((unsigned)grid), dim3(256), 0, s, mode, fmap,                \
                       static_cast<const T *>(src.ptr), src.strides[0], src.strides[1], src.strides[2],            \
                       static_cast<T *>(const_cast<void *>(dst.ptr)), dst.strides[0], dst.strides[1], dst.strides[2], \
                       (int)H, N, (int)D, total)
    if (dtype == FLA_DTYPE_BF16)
        e = vec ? FLA_FEATURE_PASS(__bf16, true) : FLA_FEATURE_PASS(__bf16, false);
    else
        e = vec ? FLA_FEATURE_PASS(_Float16, true) : FLA_FEATURE_PASS(_Float16, false);
#undef FLA_FEATURE_PASS
    return e == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
}

// ---- chunk-wise evaluation, in three steps per product:
//   chunk_states: per-chunk Y_c^T Z_c in fp32, then the exclusive running sum over the chunks
//                 before (lower) / after (upper) each chunk, rounded to the storage dtype;
//   chunk_main:   diagonal blocks plus X_c . S_c, S_c taken as stored or transposed.

// true when (x, y, z, out) of these widths can be evaluated chunk-wise: a fast kernel exists,
// the operands qualify for it, and there is more than one chunk
bool chunkable(const TriParams &p, int64_t dc, int64_t dout, int64_t N) {
    const int rows = chunk_rows(dc, dout);
    return rows != 0 && N > rows && fla::fast_path_ok(p);
}

int chunk_states(const View &y, const View &z, int64_t B, int64_t H, int64_t N, int64_t dc, int64_t dout, int upper,
                 int dtype, float *w, void *state, void *stream, int map_y = 0, const View *ymap_out = nullptr) {
    const int64_t rows = chunk_rows(dc, dout), chunks = (N + rows - 1) / rows, E = padded(dc) * padded(dout);
    hipStream_t s = static_cast<hipStream_t>(stream);
    fla::ChunkStateParams cp;
    cp.y = y.ptr, cp.z = z.ptr, cp.w = w;
    cp.ys_b = y.strides[0], cp.ys_h = y.strides[1], cp.ys_n = y.strides[2];
    cp.zs_b = z.strides[0], cp.zs_h = z.strides[1], cp.zs_n = z.strides[2];
    cp.H = (int32_t)H, cp.N = (int32_t)N, cp.BH = (int32_t)(B * H), cp.dc = (int32_t)dc, cp.dout = (int32_t)dout;
    cp.n_chunks = (int32_t)chunks;
    cp.map_y = map_y, cp.ymap_out = nullptr;
    cp.yo_b = cp.yo_h = cp.yo_n = 0;
    if (map_y) {
        cp.ymap_out = const_cast<void *>(ymap_out->ptr);
        cp.yo_b = ymap_out->strides[0], cp.yo_h = ymap_out->strides[1], cp.yo_n = ymap_out->strides[2];
    }
    if (lookup_state(dtype, dc, dout)(cp, s) != hipSuccess) return FLA_ERR_LAUNCH;
    const hipError_t e = dtype == FLA_DTYPE_BF16
                             ? fla::launch_chunk_scan<__bf16>(w, state, B * H, (int)chunks, E, upper ? 1 : 0, s)
                             : fla::launch_chunk_scan<_Float16>(w, state, B * H, (int)chunks, E, upper ? 1 : 0, s);
    return e == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
}

int chunk_main(TriParams p, int64_t dc, int64_t dout, int dtype, const void *state, int transposed, void *stream) {
    p.state = state;
    p.state_transposed = transposed;
    const hipError_t e = lookup(dtype, dc, dout)(p, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? FLA_OK : e == hipErrorNotSupported ? FLA_ERR_UNSUPPORTED : FLA_ERR_LAUNCH;
}

// Out *= phi'(x) from y = phi(x) held in `y` (Out's shape): the chain rule in the kernel's epilogue
void set_output_slope(TriParams &p, int fmap, const View &y) {
    p.map_out = fmap, p.omap = y.ptr;
    p.ms_b = y.strides[0], p.ms_h = y.strides[1], p.ms_n = y.strides[2];
}

// Out = mask(X Y^T) Z evaluated chunk-wise; same arguments as run_tri plus the workspace.
// Falls back to the quadratic kernels when the operands do not qualify for the fast path
// or the sequence is a single chunk.
int run_tri_chunked(const View &x, const View &y, const View &z, const View &out, int64_t B, int64_t H, int64_t N,
                    int64_t dc, int64_t dout, int upper, int dtype, void *workspace, int64_t workspace_bytes,
                    void *stream) {
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    if (dout > 128 && (dc <= 64 || dc > 128)) {
        const View z_hi{static_cast<const char *>(z.ptr) + 128 * 2, z.strides};
        const View out_hi{static_cast<const char *>(out.ptr) + 128 * 2, out.strides};
        if (int rc = run_tri_chunked(x, y, z, out, B, H, N, dc, 128, upper, dtype, workspace, workspace_bytes, stream))
            return rc;
        return run_tri_chunked(x, y, z_hi, out_hi, B, H, N, dc, dout - 128, upper, dtype, workspace, workspace_bytes,
                               stream);
    }
    const TriParams p = make_params(x, y, z, out, B, H, N, dc, dout, upper);
    if (!chunkable(p, dc, dout, N)) return run_tri(x, y, z, out, B, H, N, dc, dout, upper, dtype, stream);
    const int64_t rows = chunk_rows(dc, dout), chunks = (N + rows - 1) / rows, E = padded(dc) * padded(dout);
    const int64_t BH = B * H;
    if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < BH * chunks * E * 6)
        return FLA_ERR_WORKSPACE;
    float *w = static_cast<float *>(workspace);
    void *state = static_cast<char *>(workspace) + BH * chunks * E * 4;
    if (int rc = chunk_states(y, z, B, H, N, dc, dout, upper, dtype, w, state, stream)) return rc;
    return chunk_main(p, dc, dout, dtype, state, 0, stream);
}

// ---- the whole operator chunk-wise, with running states shared between products.  With equal
// padded head dims up to 128 all four products run the same square kernel, and
//     state(dQ) = state(O)^T   (sum of K_c^T V_c over the chunks before)
//     state(dK) = state(dV)^T  (sum of Q_c^T dO_c over the chunks after)
// so forward can hand its state to backward, and backward computes one new state instead of
// three.  Any other shape evaluates each product on its own.

// ---- equal padded head dims up to 128: the walk kernels (fla_chunk_walk.h).  A workgroup walks a
// segment of chunks (128 rows, 64 at D = 128) with the running state in registers; segment entry
// states come from a totals kernel and a scan over the segments.
//   D <= 64: two workgroups per CU; forward saves the 16-bit state at the entry of every chunk, and
//            one backward kernel computes dQ, dV and dK of a chunk from one set of tiles;
//   D = 128 (`split`): one workgroup per CU with two sets of tiles.  A per-chunk state would cost as
//            much traffic as an operand, so forward hands over its segments' fp32 entry states
//            only; backward is a forward-direction walk for dQ (from those entry states,
//            transposed) and a reverse walk for dK and dV.  The totals kernel visits a part of the
//            sequence only (the last segment's total is never needed).
struct WalkPlan {
    bool ok, split;
    int D, rows;
    int64_t n_chunks, seg_chunks, n_seg;  // the walks' segments
    int64_t entry_bytes;                  // fp32 entry states of the walk segments (formed in place over their totals)
    int64_t work_bytes;                   // workspace of one direction: the same
    int64_t saved_bytes;                  // what forward hands to backward: the entry states and, behind them, the state
                                          // after the last chunk of every (b, h); with the normaliser at padded head dims
                                          // up to 64, the 16-bit state of every chunk (room for the larger of the two)
};

// `mixed`: also for head dims whose padded widths differ (128 / 64, 64 / 32, 64 / 128 ...), at the larger one: the tiles
// are padded with zeros as they land in LDS, and at D = 128 the kernels built for at most 64 true columns on one side
// leave the padding's MFMAs out.  The plain operator only (the normaliser's and the feature maps' variants of the
// kernels are built for equal padded widths).
WalkPlan walk_plan(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv, bool mixed = false) {
    WalkPlan w{};
    if (B <= 0 || H <= 0 || N <= 0) return w;  // (an empty problem has no plan; the callers return before any launch)
    const int64_t wider = padded(dqk) > padded(dv) ? padded(dqk) : padded(dv);
    if (wider > 128 || (!mixed && pad_index(dqk) != pad_index(dv))) return w;
    w.D = (int)wider;
    w.rows = fla::walk_rows(w.D);
    w.split = w.D > 64;
    w.ok = N > (w.split ? 256 : w.rows);  // (D = 128: up to 256 rows one diagonal block of the quadratic kernel does it)
    if (!w.ok) return w;
    w.n_chunks = (N + w.rows - 1) / w.rows;
    // Segments per (b, h): the largest number that keeps B H n_seg within the workgroups that run at once (one per
    // CU at D = 128, two below; measured at B H = 16, N = 32768, D = 64: 256 / 512 / 1024 / 2048 workgroups give
    // 0.265 / 0.231 / 0.243 / 0.268 ms per forward + backward).  Workgroups beyond those wait for a free CU and run
    // as a second round: B H = 192, N = 4096, D = 128 takes 0.87 ms with two unequal segments in 384 workgroups
    // and 0.53 ms with one segment each; plans of several rounds of shorter segments, chosen by a cost model of
    // rounds x segment length, measured 5 to 35 % slower than this rule over B H = 65 ... 300.
    // (totals over finer segments than the walk's, 2 or 4 per walk segment, would put more workgroups on the
    // totals kernel; measured at D = 128 over B H = 8 ... 256, N = 1024 ... 32768, one total per walk segment
    // is the fastest everywhere, by 3 to 27 % of a forward + backward step)
    const int64_t resident = w.split ? 256 : 512;
    int64_t segs = resident / (B * H) > 1 ? resident / (B * H) : 1;
    if (segs > w.n_chunks) segs = w.n_chunks;
    w.seg_chunks = (w.n_chunks + segs - 1) / segs;
    w.n_seg = (w.n_chunks + w.seg_chunks - 1) / w.seg_chunks;
    w.entry_bytes = B * H * w.n_seg * w.D * w.D * 4;
    w.work_bytes = w.entry_bytes;  // (a single segment needs them only with a feature map)
    // (padded head dims up to 64: the per-chunk states of the normalised operator are the larger of the two)
    const int64_t states = w.entry_bytes + B * H * w.D * w.D * 4, per_chunk = B * H * w.n_chunks * w.D * w.D * 2;
    w.saved_bytes = w.split || states > per_chunk ? states : per_chunk;
    return w;
}

// totals of Y^T Z over the walk's segments into `work`, then the segments' entry states: their sums
// over the segments before (reverse == 0) or after (reverse != 0), written to `entry` (null: over
// the totals in `work`).  Returns where the entry states are.
// `second`: the same for another Y operand of the same layout against the same Z (the other half of a
// wide q / k) in the same launches -- one totals launch and one scan for the two of them.
struct EntryHalf {
    const void *y;  // Y's pointer (Y's strides are the first operand's)
    int64_t dy;
    void *work;
    float *entry;
    const float **where;
};

int walk_entry_states(const WalkPlan &w, const View &y, const View &z, int64_t B, int64_t H, int64_t N, int64_t dy,
                      int64_t dz, int dtype, int reverse, void *work, float *entry, const float **where, hipStream_t s,
                      int map_y = 0, const View *ymap_out = nullptr, const EntryHalf *second = nullptr,
                      bool totals_only = false) {
    fla::WalkTotalsParams tp{};
    if (map_y) {
        tp.map_y = map_y, tp.ymap_out = const_cast<void *>(ymap_out->ptr);
        tp.yo_b = ymap_out->strides[0], tp.yo_h = ymap_out->strides[1], tp.yo_n = ymap_out->strides[2];
    }
    float *totals = static_cast<float *>(work);
    if (!entry) entry = totals;
    // (two segments: the one total needed is the other segment's entry state; the totals kernel writes it as the
    // walks read it, two partial sums, and no scan follows.  A few segments more: the walks add up the totals
    // themselves as they start -- fla::walk_entries_are_totals -- and no scan follows either)
    // (totals_only: the caller's walk adds them up itself -- WalkParams::init_is_totals; not with two segments)
    const bool direct = w.n_seg == 2;
    const bool summed_on_load = fla::walk_entries_are_totals(w.D, (int)w.n_seg) || (totals_only && !direct);
    const bool no_scan = direct || summed_on_load;
    tp.y = y.ptr, tp.z = z.ptr, tp.totals = no_scan ? entry : totals, tp.direct = direct;
    tp.ys_b = y.strides[0], tp.ys_h = y.strides[1], tp.ys_n = y.strides[2];
    tp.zs_b = z.strides[0], tp.zs_h = z.strides[1], tp.zs_n = z.strides[2];
    tp.H = (int32_t)H, tp.N = (int32_t)N, tp.BH = (int32_t)(B * H), tp.dy = (int32_t)dy, tp.dz = (int32_t)dz;
    tp.n_chunks = (int32_t)w.n_chunks, tp.seg_chunks = (int32_t)w.seg_chunks, tp.n_seg = (int32_t)w.n_seg;
    // the total of the walk's last segment (first, walking in reverse) is under no sum; a feature map
    // is applied by this kernel, which then has to visit every row
    tp.seg_lo = reverse && !map_y ? 1 : 0;
    tp.seg_hi = (int32_t)(!reverse && !map_y ? w.n_seg - 1 : w.n_seg);
    if (direct) tp.seg_lo = reverse ? 1 : 0, tp.seg_hi = tp.seg_lo + 1;  // (the needed one)
    float *totals2 = nullptr, *entry2 = nullptr;
    if (second) {
        totals2 = static_cast<float *>(second->work);
        entry2 = second->entry ? second->entry : totals2;
        tp.y2 = second->y, tp.dy2 = (int32_t)second->dy, tp.totals2 = no_scan ? entry2 : totals2;
        *second->where = entry2;
    }
    if (fla::walk_totals(dtype, w.D, tp, s) != hipSuccess) return FLA_ERR_LAUNCH;
    *where = entry;
    if (no_scan) return FLA_OK;
    return fla::walk_scan(totals, entry, B * H, (int)w.n_seg, w.D, fla::walk_totals_cols(w.D, (int)dy, (int)dz), reverse,
                          s, totals2, entry2) == hipSuccess
               ? FLA_OK
               : FLA_ERR_LAUNCH;
}

// Entry states of both 128-column halves of a wide q / k (Y = the halves of `y`, against the same Z):
// one totals launch and one scan for the two when both halves take the same kernel variant, else
// one after the other.  work[h], entry[h] (null: over work[h]) and where[h] per half.
int wide_entry_states(const WalkPlan &wp, const View &y, const View &z, int64_t B, int64_t H, int64_t N, int64_t dy_all,
                      int64_t dz, int dtype, int reverse, void *const (&work)[2], float *const (&entry)[2],
                      const float *(&where)[2], hipStream_t s, bool totals_only = false) {
    const View y1{static_cast<const char *>(y.ptr) + 128 * 2, y.strides};
    const int64_t dy1 = dy_all - 128;
    if (fla::walk_totals_cols(wp.D, 128, (int)dz) == fla::walk_totals_cols(wp.D, (int)dy1, (int)dz)) {
        const EntryHalf other{y1.ptr, dy1, work[1], entry[1], &where[1]};
        return walk_entry_states(wp, y, z, B, H, N, 128, dz, dtype, reverse, work[0], entry[0], &where[0], s, 0, nullptr,
                                 &other, totals_only);
    }
    if (int rc = walk_entry_states(wp, y, z, B, H, N, 128, dz, dtype, reverse, work[0], entry[0], &where[0], s, 0, nullptr,
                                   nullptr, totals_only))
        return rc;
    return walk_entry_states(wp, y1, z, B, H, N, dy1, dz, dtype, reverse, work[1], entry[1], &where[1], s, 0, nullptr,
                             nullptr, totals_only);
}

// The normaliser's terms handed to the walk kernels (fla_chunk_walk.h, WalkParams::denom ...).
struct WalkNorm {
    float *denom;     // forward: receives n
    float eps;
    const float *dn;  // backward: dn_i = -(g_i . out_i) / n_i (and the grad_out operand holds g / n)
    void *vec;        // scratch, 2 * walk_vec_bytes(): zc, rc
    bool fused;       // out: the kernels took the terms (false: the caller runs the passes of fla_norm.h)
    bool dk_pending;  // out: ... all but dK's sum over later rows (and dK's slope, with a feature map)
};

int64_t walk_vec_bytes(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv) {
    const WalkPlan w = walk_plan(B, H, N, dqk, dv);
    return w.ok ? B * H * w.n_chunks * w.D * 4 : 0;
}

// out[bh][c] = sum over the rows before (reverse: after) chunk c of w[row] y[row] (w null: y[row])
int walk_chunk_vectors(const WalkPlan &wp, const View &y, int64_t width, const float *w, int reverse, float *out,
                       int64_t B, int64_t H, int64_t N, int dtype, hipStream_t s) {
    fla::WalkVecParams vp{};
    vp.y = y.ptr, vp.ys_b = y.strides[0], vp.ys_h = y.strides[1], vp.ys_n = y.strides[2];
    vp.w = w, vp.H = (int32_t)H, vp.N = (int32_t)N, vp.width = (int32_t)width, vp.n_chunks = (int32_t)wp.n_chunks;
    vp.out = out;
    if (fla::walk_vec_sums(dtype, wp.D, vp, B * H, s) != hipSuccess) return FLA_ERR_LAUNCH;
    return fla::walk_vec_scan(out, B * H, (int)wp.n_chunks, wp.D, reverse, s) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
}

bool states_shareable(int64_t dqk, int64_t dv, int64_t N) {
    if (pad_index(dqk) != pad_index(dv) || padded(dqk) > 128) return false;
    const int rows = chunk_rows(dqk, dv);
    return rows != 0 && N > rows;
}

// bytes of one rounded running state / of the scratch one state computation needs (fp32 chunk states)
// ---- D_qk in (128, 256] with D_v <= 128 (the small-V operator's shapes).  The scores are a sum over
// the two 128-column halves of q and k and everything is linear in them:
//     O  = tril(Q_0 K_0^T) V + tril(Q_1 K_1^T) V        dV = the same sum of the halves' dV
//     dQ_h = tril(dO V^T) K_h                           dK_h = triu(V dO^T) Q_h
// so each half runs the D = 128 walk kernels on column views of q, k, dq, dk (v and dO are padded
// with zeros in LDS, never in memory); the second half's walk adds its O (its part of dV) to what the
// first one wrote.  Forward hands over both halves' entry and final states, and backward of a half
// is then one reverse walk; without them it is the forward-direction walk for dQ_h and the dK / dV
// walk, whose second dV goes to a scratch tensor that one element-wise pass adds.
struct WidePlan {
    bool ok;
    WalkPlan wp;         // the plan of a 128 / 128 problem of the same B, H, N
    int64_t temp_bytes;  // the second half's dV in backward without forward's states, contiguous (B, H, N, D_v)
};

WidePlan wide_plan(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv) {
    WidePlan w{};
    if (dqk <= 128 || dqk > 256 || dv > 128) return w;
    w.wp = walk_plan(B, H, N, 128, 128);
    w.ok = w.wp.ok;
    w.temp_bytes = (B * H * N * dv * 2 + 255) / 256 * 256;
    return w;
}

View column_half(const View &t, int h) { return View{static_cast<const char *>(t.ptr) + h * 128 * 2, t.strides}; }

// ---- D_v in (128, 256].  O and dV are column by column in v's (dO's) columns, and dQ, dK
// are sums over them: the two column halves of v (128 and D_v - 128 columns) each run the plan of a
// (D_qk, at most 128) problem -- the walk kernels at D = 128, or the walks over a wide q / k -- on column views
// of v, O, dO, dV; the second half's dQ and dK go to scratch tensors that one element-wise pass each adds to the
// first half's.  (q and k are read once per half; the 256-row chunk kernels with their per-chunk states in
// memory, which these shapes took before, measured 2.4x slower at 256 / 256.)
struct VSplit {
    bool ok;
    int64_t dv1;         // columns of the second half
    int64_t state0;      // bytes of the first half's state (the second half's follows it)
    int64_t temp_bytes;  // one scratch tensor, contiguous (B, H, N, D_qk)
};

int64_t shared_state_bytes(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv);
int64_t chunked_op_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv);

VSplit vsplit_plan(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv) {
    VSplit s{};
    if (dv <= 128 || dv > 256 || dqk < 1 || dqk > 256 || B <= 0 || H <= 0) return s;
    s.dv1 = dv - 128;
    auto planned = [&](int64_t d) { return walk_plan(B, H, N, dqk, d, true).ok || wide_plan(B, H, N, dqk, d).ok; };
    s.ok = planned(128) && planned(s.dv1);
    if (!s.ok) return s;
    s.state0 = (shared_state_bytes(B, H, N, dqk, 128) + 255) / 256 * 256;
    s.temp_bytes = (B * H * N * dqk * 2 + 255) / 256 * 256;
    return s;
}

View v_half(const View &t, int j) { return View{static_cast<const char *>(t.ptr) + j * 128 * 2, t.strides}; }

// what the halves' own calls use of the workspace (the scratch tensors follow it)
int64_t vsplit_inner_bytes(const VSplit &vs, int64_t B, int64_t H, int64_t N, int64_t dqk) {
    const int64_t a = chunked_op_workspace_bytes(B, H, N, dqk, 128), b = chunked_op_workspace_bytes(B, H, N, dqk, vs.dv1);
    return ((a > b ? a : b) + 255) / 256 * 256;
}

int64_t state_core_bytes(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv) {
    if (const VSplit vs = vsplit_plan(B, H, N, dqk, dv); vs.ok) return vs.state0 + shared_state_bytes(B, H, N, dqk, vs.dv1);
    const WalkPlan w = walk_plan(B, H, N, dqk, dv, true);
    if (w.ok && !w.split) return w.saved_bytes;  // one state per 128-row chunk (also room for the 256-row chunks' states)
    if (!states_shareable(dqk, dv, N)) {
        const WidePlan wide = wide_plan(B, H, N, dqk, dv);
        return wide.ok ? 2 * wide.wp.saved_bytes : w.ok ? w.saved_bytes : 0;
    }
    const int64_t rows = chunk_rows(dqk, dv);
    const int64_t per_chunk = B * H * ((N + rows - 1) / rows) * padded(dqk) * padded(dv) * 2;
    return w.ok && w.saved_bytes > per_chunk ? w.saved_bytes : per_chunk;  // (split: either path's state fits)
}

// The buffer forward's state goes to: the states above and, behind them, room for the running sums of
// k at the entry of every chunk, which the normalised forward leaves there for its backward.
int64_t shared_state_bytes(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv) {
    const int64_t core = state_core_bytes(B, H, N, dqk, dv);
    return core ? core + walk_vec_bytes(B, H, N, dqk, dv) : 0;
}

// workspace of the two-halves evaluation: the scratch tensor for dV, then totals and entry states of both
// halves (two sets of them in backward: Q^T dO, and K^T V when forward's entry states are not given)
int64_t wide_workspace_bytes(const WidePlan &w) { return w.temp_bytes + 4 * w.wp.work_bytes; }

int64_t chunked_op_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv) {
    const int64_t shared = shared_state_bytes(B, H, N, dqk, dv);
    if (shared) {  // fp32 chunk states (2x) + two rounded states (backward without a saved one); the walk's totals
        const WalkPlan w = walk_plan(B, H, N, dqk, dv, true);
        if (w.ok || states_shareable(dqk, dv, N)) {
            int64_t m = w.ok && w.work_bytes * 2 > shared * 4 ? w.work_bytes * 2 : shared * 4;
            if (pad_index(dqk) != pad_index(dv)) {  // (off the walks these shapes evaluate product by product)
                const int64_t a = chunked_bytes(B, H, N, dqk, dv), b = chunked_bytes(B, H, N, dv, dqk);
                m = a > m ? a : m, m = b > m ? b : m;
            }
            return m;
        }
    }
    int64_t m = chunked_bytes(B, H, N, dqk, dv);
    const int64_t t = chunked_bytes(B, H, N, dv, dqk);
    if (t > m) m = t;
    const WidePlan wide = wide_plan(B, H, N, dqk, dv);
    if (wide.ok && wide_workspace_bytes(wide) > m) m = wide_workspace_bytes(wide);
    if (const VSplit vs = vsplit_plan(B, H, N, dqk, dv); vs.ok) {
        const int64_t need = vsplit_inner_bytes(vs, B, H, N, dqk) + 2 * vs.temp_bytes;
        if (need > m) m = need;
    }
    return m;
}

// the walk that computes out = lower(x y^T) z + x S with S += y^T z (fla::walk_fwd_kernel's roles)
fla::WalkParams lower_walk_params(const WalkPlan &wp, const View &x, const View &y, const View &z, const View &out,
                                  int64_t B, int64_t H, int64_t N, int64_t wxy, int64_t wz, const float *entry) {
    fla::WalkParams w{};
    w.q = x.ptr, w.k = y.ptr, w.v = z.ptr, w.o = const_cast<void *>(out.ptr);
    w.qs_b = x.strides[0], w.qs_h = x.strides[1], w.qs_n = x.strides[2];
    w.ks_b = y.strides[0], w.ks_h = y.strides[1], w.ks_n = y.strides[2];
    w.vs_b = z.strides[0], w.vs_h = z.strides[1], w.vs_n = z.strides[2];
    w.os_b = out.strides[0], w.os_h = out.strides[1], w.os_n = out.strides[2];
    w.H = (int32_t)H, w.N = (int32_t)N, w.BH = (int32_t)(B * H), w.wqk = (int32_t)wxy, w.wv = (int32_t)wz;
    w.n_chunks = (int32_t)wp.n_chunks, w.seg_chunks = (int32_t)wp.seg_chunks, w.n_seg = (int32_t)wp.n_seg;
    w.init = wp.n_seg > 1 ? entry : nullptr;
    return w;
}

bool wide_fast_path(const View &q, const View &k, const View &v, const View &o, int64_t B, int64_t H, int64_t N,
                    int64_t dqk, int64_t dv) {
    return fla::fast_path_ok(make_params(q, k, v, o, B, H, N, 128, dv, 0)) &&
           fla::fast_path_ok(make_params(column_half(q, 1), column_half(k, 1), v, o, B, H, N, dqk - 128, dv, 0));
}

int wide_forward(const WidePlan &wide, const View &q, const View &k, const View &v, const View &o, int64_t B, int64_t H,
                 int64_t N, int64_t dqk, int64_t dv, int dtype, void *state_out, void *workspace, hipStream_t s) {
    const WalkPlan &wp = wide.wp;
    char *ws = static_cast<char *>(workspace);
    const float *entry[2] = {nullptr, nullptr};
    // A few segments more than two: no scan -- the walk adds up the totals of the segments before its own as it
    // starts (three of each half in flight together) and writes the entry state it formed for backward
    // (B 4, H 16, N 4096, D_qk 256, D_v 64, four segments: 0.273 -> 0.267 ms per forward + backward, and 0.264 with
    // the reverse walk doing the same).
    const bool sum_on_load = wp.n_seg >= 3 && wp.n_seg <= 7;
    float *keep[2] = {nullptr, nullptr};
    if (wp.n_seg > 1) {
        // (kept for backward when there is a state buffer: each half's entry states, its final state behind them;
        // otherwise, and the totals that the walk adds up, in the workspace behind the scratch tensor)
        void *work[2];
        for (int h = 0; h < 2; ++h) {
            if (state_out) keep[h] = reinterpret_cast<float *>(static_cast<char *>(state_out) + h * wp.saved_bytes);
            work[h] = keep[h] && !sum_on_load ? static_cast<void *>(keep[h])
                                              : static_cast<void *>(ws + wide.temp_bytes + h * wp.work_bytes);
        }
        float *const none[2] = {nullptr, nullptr};
        if (int rc = wide_entry_states(wp, k, v, B, H, N, dqk, dv, dtype, 0, work, sum_on_load ? none : keep, entry, s,
                                       sum_on_load))
            return rc;
    }
    // one walk over both halves (the second one's columns start 128 elements into q's and k's rows)
    fla::WalkParams w = lower_walk_params(wp, q, k, v, o, B, H, N, 128, dv, entry[0]);
    w.wqk2 = (int32_t)(dqk - 128), w.init2 = wp.n_seg > 1 ? entry[1] : nullptr;
    if (sum_on_load) w.init_is_totals = 1, w.entry_out = keep[0], w.entry_out2 = keep[1];
    if (state_out) {  // (behind each half's entry states: its state after the last chunk)
        w.total_out = reinterpret_cast<float *>(static_cast<char *>(state_out) + wp.entry_bytes);
        w.total_out2 = reinterpret_cast<float *>(static_cast<char *>(state_out) + wp.saved_bytes + wp.entry_bytes);
    }
    return fla::walk_fwd_wide(dtype, w, s) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
}

int wide_backward(const WidePlan &wide, const View &go, const View &q, const View &k, const View &v, const View &dq,
                  const View &dk, const View &dvv, int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv, int dtype,
                  const void *state_in, void *workspace, hipStream_t s) {
    const WalkPlan &wp = wide.wp;
    char *ws = static_cast<char *>(workspace);
    const int64_t temp_strides[4] = {H * N * dv, N * dv, dv, 1};
    const View temp{ws, temp_strides};
    // entry states of both halves up front: Q_h^T dO over the segments after, and -- when forward's are not
    // at hand -- K_h^T V over the segments before
    const float *fwd_entries[2] = {nullptr, nullptr}, *entries[2] = {nullptr, nullptr};
    // (the reverse walks add up the totals of the segments after their own themselves, as forward does)
    const bool rev_sums_on_load = state_in && wp.n_seg >= 3 && wp.n_seg <= 7;
    if (wp.n_seg > 1) {
        float *const none[2] = {nullptr, nullptr};
        char *base = ws + wide.temp_bytes;
        if (state_in) {
            for (int h = 0; h < 2; ++h)
                fwd_entries[h] = reinterpret_cast<const float *>(static_cast<const char *>(state_in) + h * wp.saved_bytes);
        } else {
            void *const work[2] = {base + 2 * wp.work_bytes, base + 3 * wp.work_bytes};
            if (int rc = wide_entry_states(wp, k, v, B, H, N, dqk, dv, dtype, 0, work, none, fwd_entries, s)) return rc;
        }
        void *const work[2] = {base, base + wp.work_bytes};
        if (int rc = wide_entry_states(wp, q, go, B, H, N, dqk, dv, dtype, 1, work, none, entries, s, rev_sums_on_load))
            return rc;
    }
    if (state_in && dv <= 64) {  // forward's states at hand, narrow v: one reverse walk over both halves
        fla::WalkParams r{};
        r.q = q.ptr, r.k = k.ptr, r.v = v.ptr, r.go = go.ptr;
        r.dq = const_cast<void *>(dq.ptr), r.dk = const_cast<void *>(dk.ptr), r.dv = const_cast<void *>(dvv.ptr);
        r.qs_b = q.strides[0], r.qs_h = q.strides[1], r.qs_n = q.strides[2];
        r.ks_b = k.strides[0], r.ks_h = k.strides[1], r.ks_n = k.strides[2];
        r.vs_b = v.strides[0], r.vs_h = v.strides[1], r.vs_n = v.strides[2];
        r.gs_b = go.strides[0], r.gs_h = go.strides[1], r.gs_n = go.strides[2];
        r.dqs_b = dq.strides[0], r.dqs_h = dq.strides[1], r.dqs_n = dq.strides[2];
        r.dks_b = dk.strides[0], r.dks_h = dk.strides[1], r.dks_n = dk.strides[2];
        r.dvs_b = dvv.strides[0], r.dvs_h = dvv.strides[1], r.dvs_n = dvv.strides[2];
        r.H = (int32_t)H, r.N = (int32_t)N, r.BH = (int32_t)(B * H), r.wqk = 128, r.wqk2 = (int32_t)(dqk - 128);
        r.wv = (int32_t)dv;
        r.n_chunks = (int32_t)wp.n_chunks, r.seg_chunks = (int32_t)wp.seg_chunks, r.n_seg = (int32_t)wp.n_seg;
        r.init = entries[0], r.init2 = entries[1], r.init_is_totals = rev_sums_on_load;
        const char *half0 = static_cast<const char *>(state_in), *half1 = half0 + wp.saved_bytes;
        r.xinit = reinterpret_cast<const float *>(half0), r.xinit2 = reinterpret_cast<const float *>(half1);
        r.xtotal = reinterpret_cast<const float *>(half0 + wp.entry_bytes);
        r.xtotal2 = reinterpret_cast<const float *>(half1 + wp.entry_bytes);
        return fla::walk_bwd_rev_wide(dtype, r, s) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
    }
    for (int h = 0; h < 2; ++h) {
        const View qh = column_half(q, h), kh = column_half(k, h), dqh = column_half(dq, h), dkh = column_half(dk, h);
        const int64_t wqk = h == 0 ? 128 : dqk - 128;
        const float *fwd_entry = fwd_entries[h], *entry = entries[h];
        const View &dvh = h == 0 ? dvv : temp;
        if (state_in) {  // forward's states at hand: dQ_h, dK_h and this half's part of dV in one reverse walk
            fla::WalkParams r{};
            r.q = qh.ptr, r.k = kh.ptr, r.v = v.ptr, r.go = go.ptr;
            r.dq = const_cast<void *>(dqh.ptr), r.dk = const_cast<void *>(dkh.ptr), r.dv = const_cast<void *>(dvv.ptr);
            r.accumulate = h;  // (the second half's walk adds its part of dV to the first one's)
            r.qs_b = qh.strides[0], r.qs_h = qh.strides[1], r.qs_n = qh.strides[2];
            r.ks_b = kh.strides[0], r.ks_h = kh.strides[1], r.ks_n = kh.strides[2];
            r.vs_b = v.strides[0], r.vs_h = v.strides[1], r.vs_n = v.strides[2];
            r.gs_b = go.strides[0], r.gs_h = go.strides[1], r.gs_n = go.strides[2];
            r.dqs_b = dqh.strides[0], r.dqs_h = dqh.strides[1], r.dqs_n = dqh.strides[2];
            r.dks_b = dkh.strides[0], r.dks_h = dkh.strides[1], r.dks_n = dkh.strides[2];
            r.dvs_b = dvv.strides[0], r.dvs_h = dvv.strides[1], r.dvs_n = dvv.strides[2];
            r.H = (int32_t)H, r.N = (int32_t)N, r.BH = (int32_t)(B * H), r.wqk = (int32_t)wqk, r.wv = (int32_t)dv;
            r.n_chunks = (int32_t)wp.n_chunks, r.seg_chunks = (int32_t)wp.seg_chunks, r.n_seg = (int32_t)wp.n_seg;
            r.init = entry, r.init_is_totals = rev_sums_on_load;
            const char *half = static_cast<const char *>(state_in) + h * wp.saved_bytes;
            r.xinit = reinterpret_cast<const float *>(half);
            r.xtotal = reinterpret_cast<const float *>(half + wp.entry_bytes);
            if (fla::walk_bwd_rev(dtype, wp.D, r, s) != hipSuccess) return FLA_ERR_LAUNCH;
            continue;
        }
        // dQ_h = lower(dO V^T) K_h + dO S_h^T: the forward walk over (dO, V, K_h)
        fla::WalkParams w = lower_walk_params(wp, go, v, kh, dqh, B, H, N, dv, wqk, fwd_entry);
        w.init_transposed = 1;
        if (fla::walk_fwd(dtype, wp.D, w, s) != hipSuccess) return FLA_ERR_LAUNCH;
        // dV (this half's part) and dK_h: the reverse walk
        fla::WalkParams r{};
        r.q = qh.ptr, r.k = kh.ptr, r.v = v.ptr, r.go = go.ptr;
        r.dk = const_cast<void *>(dkh.ptr), r.dv = const_cast<void *>(dvh.ptr);
        r.qs_b = qh.strides[0], r.qs_h = qh.strides[1], r.qs_n = qh.strides[2];
        r.ks_b = kh.strides[0], r.ks_h = kh.strides[1], r.ks_n = kh.strides[2];
        r.vs_b = v.strides[0], r.vs_h = v.strides[1], r.vs_n = v.strides[2];
        r.gs_b = go.strides[0], r.gs_h = go.strides[1], r.gs_n = go.strides[2];
        r.dks_b = dkh.strides[0], r.dks_h = dkh.strides[1], r.dks_n = dkh.strides[2];
        r.dvs_b = dvh.strides[0], r.dvs_h = dvh.strides[1], r.dvs_n = dvh.strides[2];
        r.H = (int32_t)H, r.N = (int32_t)N, r.BH = (int32_t)(B * H), r.wqk = (int32_t)wqk, r.wv = (int32_t)dv;
        r.n_chunks = (int32_t)wp.n_chunks, r.seg_chunks = (int32_t)wp.seg_chunks, r.n_seg = (int32_t)wp.n_seg;
        r.init = entry;
        if (fla::walk_dkdv(dtype, wp.D, r, s) != hipSuccess) return FLA_ERR_LAUNCH;
    }
    return state_in ? FLA_OK : launch_feature_pass(3, 0, temp, dvv, B, H, N, dv, dtype, s);
}

// both column halves of (x4, o4) = (v, O) / (dO, dV) with (a, b) = (q, k) / (dQ, dK) qualify for their plans' kernels
bool vsplit_fast_path(const VSplit &vs, const View &a, const View &b, const View &x4, const View &o4, int64_t B, int64_t H,
                      int64_t N, int64_t dqk) {
    for (int j = 0; j < 2; ++j) {
        const int64_t d = j == 0 ? 128 : vs.dv1;
        const View xj = v_half(x4, j), oj = v_half(o4, j);
        const bool ok = dqk > 128 ? wide_fast_path(a, b, xj, oj, B, H, N, dqk, d)
                                  : fla::fast_path_ok(make_params(a, b, xj, oj, B, H, N, dqk, d, 0));
        if (!ok) return false;
    }
    return true;
}

int chunked_forward(const View &q, const View &k, const View &v, const View &o, int64_t B, int64_t H, int64_t N,
                    int64_t dqk, int64_t dv, int dtype, void *state_out, int32_t *state_valid, void *workspace,
                    int64_t workspace_bytes, void *stream, int fmap, const View *mapped, bool *mapped_done, WalkNorm *nx);
int chunked_backward(const View &go, const View &q, const View &k, const View &v, const View &dq, const View &dk,
                     const View &dvv, int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv, int dtype,
                     const void *state_in, void *workspace, int64_t workspace_bytes, void *stream, int fmap, WalkNorm *nx);

// fmap != 0 (feature_forward below): q and k hold the arguments xq, xk of the feature map phi, and
// `mapped` = {phi(xq), phi(xk)} are outputs: the state kernel maps xk as it loads it and writes
// phi(xk), which the main kernel then reads as its Y operand; the main kernel maps its X rows xq
// and writes phi(xq).  Only the shared-state fast path does this; *mapped_done says whether it ran.
int chunked_forward(const View &q, const View &k, const View &v, const View &o, int64_t B, int64_t H, int64_t N,
                    int64_t dqk, int64_t dv, int dtype, void *state_out, int32_t *state_valid, void *workspace,
                    int64_t workspace_bytes, void *stream, int fmap = 0, const View *mapped = nullptr,
                    bool *mapped_done = nullptr, WalkNorm *nx = nullptr) {
    if (state_valid) *state_valid = 0;
    if (nx) nx->fused = nx->dk_pending = false;
    const View all[] = {q, k, v, o};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (int rc = check_alias_fwd(q, k, v, o, B, H, N, dqk, dv)) return rc;
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    if (!fmap && !nx) {
        // a v wider than 128 columns: its two column halves, one after the other (the second half's state behind the first's)
        const VSplit vs = vsplit_plan(B, H, N, dqk, dv);
        if (vs.ok && vsplit_fast_path(vs, q, k, v, o, B, H, N, dqk)) {
            if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 ||
                workspace_bytes < vsplit_inner_bytes(vs, B, H, N, dqk))
                return FLA_ERR_WORKSPACE;
            if (state_out && reinterpret_cast<uintptr_t>(state_out) % 16 != 0) return FLA_ERR_WORKSPACE;
            int32_t valid[2] = {0, 0};
            for (int j = 0; j < 2; ++j) {
                void *st = state_out ? static_cast<char *>(state_out) + j * vs.state0 : nullptr;
                if (int rc = chunked_forward(q, k, v_half(v, j), v_half(o, j), B, H, N, dqk, j == 0 ? 128 : vs.dv1, dtype, st,
                                             &valid[j], workspace, workspace_bytes, stream, 0, nullptr, nullptr, nullptr))
                    return rc;
            }
            if (state_out && state_valid) *state_valid = valid[0] && valid[1];
            return FLA_OK;
        }
        const WidePlan wide = wide_plan(B, H, N, dqk, dv);
        if (wide.ok && wide_fast_path(q, k, v, o, B, H, N, dqk, dv)) {
            if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < wide_workspace_bytes(wide))
                return FLA_ERR_WORKSPACE;
            if (state_out && reinterpret_cast<uintptr_t>(state_out) % 16 != 0) return FLA_ERR_WORKSPACE;
            if (int rc = wide_forward(wide, q, k, v, o, B, H, N, dqk, dv, dtype, state_out, workspace,
                                      static_cast<hipStream_t>(stream)))
                return rc;
            if (state_out && state_valid) *state_valid = 1;
            return FLA_OK;
        }
    }
    const WalkPlan wp = walk_plan(B, H, N, dqk, dv, !fmap && !nx);
    if (wp.ok && fla::fast_path_ok(make_params(q, k, v, o, B, H, N, dqk, dv, 0)) &&
        (!fmap || fla::fast_path_ok(make_params(mapped[0], mapped[1], v, o, B, H, N, dqk, dv, 0)))) {
        // the segments' entry states; with a feature map the same kernel maps xk as it loads it and
        // writes phi(xk), which the walk then reads (so it runs for a single segment as well)
        const bool need_totals = wp.n_seg > 1 || fmap;
        // the entry states (and the state after the last chunk) are what backward gets, so the scan writes
        // them to state_out (the totals themselves are computed there, and no workspace is used);
        // the normalised operator at padded head dims up to 64 hands over the 16-bit state of every chunk instead
        const bool in_state = state_out && (wp.split || !nx);
        // D = 128, a few segments more than two: the totals go to the workspace, the walk adds them up itself as it starts
        // and writes the entry states it formed to state_out -- no scan launch (B H 64, N 4096: see wide_forward)
        const bool sum_on_load = wp.split && !fmap && !nx && wp.n_seg >= 3 && wp.n_seg <= 7;
        if (need_totals && (!in_state || sum_on_load) &&
            (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < wp.work_bytes))
            return FLA_ERR_WORKSPACE;
        if (state_out && reinterpret_cast<uintptr_t>(state_out) % 16 != 0) return FLA_ERR_WORKSPACE;
        hipStream_t s = static_cast<hipStream_t>(stream);
        const float *entry = nullptr;
        if (need_totals)
            if (int rc = walk_entry_states(wp, k, v, B, H, N, dqk, dv, dtype, 0,
                                           in_state && !sum_on_load ? state_out : workspace,
                                           in_state && !sum_on_load ? static_cast<float *>(state_out) : nullptr, &entry, s,
                                           fmap, fmap ? &mapped[1] : nullptr, nullptr, sum_on_load))
                return rc;
        const View &kk = fmap ? mapped[1] : k;
        fla::WalkParams w{};
        if (fmap) {
            w.fmap = fmap, w.qmap_out = const_cast<void *>(mapped[0].ptr);
            w.qo_b = mapped[0].strides[0], w.qo_h = mapped[0].strides[1], w.qo_n = mapped[0].strides[2];
        }
        w.q = q.ptr, w.k = kk.ptr, w.v = v.ptr, w.o = const_cast<void *>(o.ptr);
        w.qs_b = q.strides[0], w.qs_h = q.strides[1], w.qs_n = q.strides[2];
        w.ks_b = kk.strides[0], w.ks_h = kk.strides[1], w.ks_n = kk.strides[2];
        w.vs_b = v.strides[0], w.vs_h = v.strides[1], w.vs_n = v.strides[2];
        w.os_b = o.strides[0], w.os_h = o.strides[1], w.os_n = o.strides[2];
        w.H = (int32_t)H, w.N = (int32_t)N, w.BH = (int32_t)(B * H), w.wqk = (int32_t)dqk, w.wv = (int32_t)dv;
        w.n_chunks = (int32_t)wp.n_chunks, w.seg_chunks = (int32_t)wp.seg_chunks, w.n_seg = (int32_t)wp.n_seg;
        w.init = wp.n_seg > 1 ? entry : nullptr, w.saved = in_state ? nullptr : state_out;
        if (sum_on_load) w.init_is_totals = 1, w.entry_out = in_state ? static_cast<float *>(state_out) : nullptr;
        if (in_state) w.total_out = reinterpret_cast<float *>(static_cast<char *>(state_out) + wp.entry_bytes);
        if (nx) {  // the normaliser inside the walk: zc = running sum of k at the entry of every chunk
            // (kept behind the state, when there is one, for backward)
            float *zc = state_out ? reinterpret_cast<float *>(static_cast<char *>(state_out) + state_core_bytes(B, H, N, dqk, dv))
                                  : static_cast<float *>(nx->vec);
            if (int rc = walk_chunk_vectors(wp, kk, dqk, nullptr, 0, zc, B, H, N, dtype, s)) return rc;
            w.denom = nx->denom, w.eps = nx->eps, w.zc = zc;
            nx->fused = true;
        }
        if (fla::walk_fwd(dtype, wp.D, w, s) != hipSuccess) return FLA_ERR_LAUNCH;
        if (mapped_done) *mapped_done = true;
        if (state_out && state_valid) *state_valid = 1;
        return FLA_OK;
    }
    TriParams p = make_params(q, fmap ? mapped[1] : k, v, o, B, H, N, dqk, dv, 0);
    // with a feature map: xk is read by the state kernel's loads, and phi(xq), phi(xk) are written with 16-byte stores
    const bool k_fast = !fmap || (fla::fast_path_ok(make_params(q, k, v, o, B, H, N, dqk, dv, 0)) &&
                                  fla::fast_path_ok(make_params(mapped[0], mapped[1], v, o, B, H, N, dqk, dv, 0)));
    if (!states_shareable(dqk, dv, N) || !fla::fast_path_ok(p) || !k_fast) {
        if (fmap) return FLA_OK;  // *mapped_done stays false: the caller maps with a pass of its own
        return run_tri_chunked(q, k, v, o, B, H, N, dqk, dv, 0, dtype, workspace, workspace_bytes, stream);
    }
    if (fmap) {
        p.map_x = fmap, p.xmap_out = const_cast<void *>(mapped[0].ptr);
        p.xo_b = mapped[0].strides[0], p.xo_h = mapped[0].strides[1], p.xo_n = mapped[0].strides[2];
    }
    const int64_t sb = shared_state_bytes(B, H, N, dqk, dv);
    if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < sb * (state_out ? 2 : 3))
        return FLA_ERR_WORKSPACE;
    if (state_out && reinterpret_cast<uintptr_t>(state_out) % 16 != 0) return FLA_ERR_WORKSPACE;
    float *w = static_cast<float *>(workspace);
    void *state = state_out ? state_out : static_cast<char *>(workspace) + 2 * sb;
    if (int rc = chunk_states(k, v, B, H, N, dqk, dv, 0, dtype, w, state, stream, fmap, fmap ? &mapped[1] : nullptr))
        return rc;
    if (int rc = chunk_main(p, dqk, dv, dtype, state, 0, stream)) return rc;
    if (mapped_done) *mapped_done = true;
    // (where the walk kernels exist, backward reads a handed-over state in THEIR format: the 256-row
    // chunks' state written here is not offered, and backward computes its own)
    if (state_out && state_valid && !wp.ok) *state_valid = 1;
    return FLA_OK;
}

int chunked_backward(const View &go, const View &q, const View &k, const View &v, const View &dq, const View &dk,
                     const View &dvv, int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv, int dtype,
                     const void *state_in, void *workspace, int64_t workspace_bytes, void *stream, int fmap = 0,
                     WalkNorm *nx = nullptr) {
    if (nx) nx->fused = nx->dk_pending = false;
    const View all[] = {go, q, k, v, dq, dk, dvv};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (int rc = check_alias_bwd(go, q, k, v, nullptr, dq, dk, dvv, B, H, N, dqk, dv)) return rc;
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    // fmap != 0: q and k hold y = phi(x) (what the forward pass wrote), and the gradients leave as
    // gradients with respect to x: dQ and dK are multiplied by phi'(x), computed from y -- in the
    // kernels' epilogue on the fast path, by a pass of its own after the products otherwise.
    TriParams pq = make_params(go, v, k, dq, B, H, N, dv, dqk, 0);   // dQ = lower(dO V^T) K
    TriParams pv = make_params(k, q, go, dvv, B, H, N, dqk, dv, 1);  // dV = upper(K Q^T) dO
    TriParams pk = make_params(v, go, q, dk, B, H, N, dv, dqk, 1);   // dK = upper(V dO^T) Q
    if (!fmap && !nx) {
        // a v wider than 128 columns: dV of each column half; dQ and dK of the second half to scratch tensors, then added
        const VSplit vs = vsplit_plan(B, H, N, dqk, dv);
        if (vs.ok && vsplit_fast_path(vs, q, k, v, go, B, H, N, dqk) && vsplit_fast_path(vs, dq, dk, dvv, dvv, B, H, N, dqk)) {
            const int64_t inner = vsplit_inner_bytes(vs, B, H, N, dqk);
            if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < inner + 2 * vs.temp_bytes)
                return FLA_ERR_WORKSPACE;
            if (state_in && reinterpret_cast<uintptr_t>(state_in) % 16 != 0) return FLA_ERR_WORKSPACE;
            const int64_t temp_strides[4] = {H * N * dqk, N * dqk, dqk, 1};
            const View tq{static_cast<char *>(workspace) + inner, temp_strides};
            const View tk{static_cast<char *>(workspace) + inner + vs.temp_bytes, temp_strides};
            for (int j = 0; j < 2; ++j) {
                const void *st = state_in ? static_cast<const char *>(state_in) + j * vs.state0 : nullptr;
                if (int rc = chunked_backward(v_half(go, j), q, k, v_half(v, j), j == 0 ? dq : tq, j == 0 ? dk : tk,
                                              v_half(dvv, j), B, H, N, dqk, j == 0 ? 128 : vs.dv1, dtype, st, workspace, inner,
                                              stream, 0, nullptr))
                    return rc;
            }
            if (int rc = launch_feature_pass(3, 0, tq, dq, B, H, N, dqk, dtype, stream)) return rc;
            return launch_feature_pass(3, 0, tk, dk, B, H, N, dqk, dtype, stream);
        }
        const WidePlan wide = wide_plan(B, H, N, dqk, dv);
        if (wide.ok && wide_fast_path(q, k, v, go, B, H, N, dqk, dv) && wide_fast_path(dq, dk, dvv, dvv, B, H, N, dqk, dv)) {
            if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < wide_workspace_bytes(wide))
                return FLA_ERR_WORKSPACE;
            if (state_in && reinterpret_cast<uintptr_t>(state_in) % 16 != 0) return FLA_ERR_WORKSPACE;
            return wide_backward(wide, go, q, k, v, dq, dk, dvv, B, H, N, dqk, dv, dtype, state_in, workspace,
                                 static_cast<hipStream_t>(stream));
        }
    }
    // (with the normaliser's terms still to be added by the caller, so is the slope)
    const int fmap_late = nx ? 0 : fmap;
    const WalkPlan wp = walk_plan(B, H, N, dqk, dv, !fmap && !nx);
    // (what forward saved is in the walks' format; at D = 128 the entry states are cheap to recompute)
    const bool walk = wp.ok && (state_in || wp.split);
    // (padded widths that differ: the walks or product by product -- the 256-row chunks share states between equal ones only)
    const bool mixed_walk = walk && pad_index(dqk) != pad_index(dv);
    if ((!states_shareable(dqk, dv, N) && !mixed_walk) || !fla::fast_path_ok(pq) || !fla::fast_path_ok(pv) ||
        !fla::fast_path_ok(pk)) {
        if (int rc = run_tri_chunked(go, v, k, dq, B, H, N, dv, dqk, 0, dtype, workspace, workspace_bytes, stream))
            return rc;
        if (int rc = run_tri_chunked(k, q, go, dvv, B, H, N, dqk, dv, 1, dtype, workspace, workspace_bytes, stream))
            return rc;
        if (int rc = run_tri_chunked(v, go, q, dk, B, H, N, dv, dqk, 1, dtype, workspace, workspace_bytes, stream))
            return rc;
        if (!fmap_late) return FLA_OK;
        if (int rc = launch_feature_pass(2, fmap, q, dq, B, H, N, dqk, dtype, stream)) return rc;
        return launch_feature_pass(2, fmap, k, dk, B, H, N, dqk, dtype, stream);
    }
    // the normalised forward left zc behind its state
    const float *zc_saved = nx && state_in ? reinterpret_cast<const float *>(static_cast<const char *>(state_in) +
                                                                           state_core_bytes(B, H, N, dqk, dv))
                                           : nullptr;
    if (walk && wp.split) {
        // workspace: totals and entry states of Q^T dO; behind them those of K^T V when forward's are not given
        if (wp.n_seg > 1 && (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 ||
                             workspace_bytes < wp.work_bytes * (state_in ? 1 : 2)))
            return FLA_ERR_WORKSPACE;
        if (state_in && reinterpret_cast<uintptr_t>(state_in) % 16 != 0) return FLA_ERR_WORKSPACE;
        hipStream_t s = static_cast<hipStream_t>(stream);
        const float *entry = nullptr;
        // with forward's states at hand (and without the normaliser): one reverse walk
        const bool one_walk = state_in && !nx;
        // (... which adds up the totals of the segments after its own itself, as forward does)
        const bool rev_sums_on_load = one_walk && wp.n_seg >= 3 && wp.n_seg <= 7;
        if (wp.n_seg > 1) {
            if (!state_in) {
                const float *fwd_entry = nullptr;
                if (int rc = walk_entry_states(wp, k, v, B, H, N, dqk, dv, dtype, 0, static_cast<char *>(workspace) + wp.work_bytes,
                                               nullptr, &fwd_entry, s))
                    return rc;
                state_in = fwd_entry;
            }
            if (int rc = walk_entry_states(wp, q, go, B, H, N, dqk, dv, dtype, 1, workspace, nullptr, &entry, s, 0, nullptr,
                                           nullptr, rev_sums_on_load))
                return rc;
        }
        float *zc = nullptr, *rcv = nullptr;
        if (nx) {  // zc: running sum of k at the entry of every chunk; rc: sum of dn_i q_i over the rows after it
            zc = static_cast<float *>(nx->vec);
            rcv = reinterpret_cast<float *>(static_cast<char *>(nx->vec) + walk_vec_bytes(B, H, N, dqk, dv));
            if (int rc = walk_chunk_vectors(wp, q, dqk, nx->dn, 1, rcv, B, H, N, dtype, s)) return rc;
            if (zc_saved) zc = const_cast<float *>(zc_saved);
            else if (int rc = walk_chunk_vectors(wp, k, dqk, nullptr, 0, zc, B, H, N, dtype, s)) return rc;
        }
        if (one_walk) {
            fla::WalkParams r{};
            r.q = q.ptr, r.k = k.ptr, r.v = v.ptr, r.go = go.ptr;
            r.dq = const_cast<void *>(dq.ptr), r.dk = const_cast<void *>(dk.ptr), r.dv = const_cast<void *>(dvv.ptr);
            r.qs_b = q.strides[0], r.qs_h = q.strides[1], r.qs_n = q.strides[2];
            r.ks_b = k.strides[0], r.ks_h = k.strides[1], r.ks_n = k.strides[2];
            r.vs_b = v.strides[0], r.vs_h = v.strides[1], r.vs_n = v.strides[2];
            r.gs_b = go.strides[0], r.gs_h = go.strides[1], r.gs_n = go.strides[2];
            r.dqs_b = dq.strides[0], r.dqs_h = dq.strides[1], r.dqs_n = dq.strides[2];
            r.dks_b = dk.strides[0], r.dks_h = dk.strides[1], r.dks_n = dk.strides[2];
            r.dvs_b = dvv.strides[0], r.dvs_h = dvv.strides[1], r.dvs_n = dvv.strides[2];
            r.H = (int32_t)H, r.N = (int32_t)N, r.BH = (int32_t)(B * H), r.wqk = (int32_t)dqk, r.wv = (int32_t)dv;
            r.n_chunks = (int32_t)wp.n_chunks, r.seg_chunks = (int32_t)wp.seg_chunks, r.n_seg = (int32_t)wp.n_seg;
            r.init = entry, r.fmap = fmap;  // (dQ, dK: the slopes from phi(xq), phi(xk) in the Q and K tiles)
            r.init_is_totals = rev_sums_on_load;
            r.xinit = static_cast<const float *>(state_in);
            r.xtotal = reinterpret_cast<const float *>(static_cast<const char *>(state_in) + wp.entry_bytes);
            return fla::walk_bwd_rev(dtype, wp.D, r, s) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
        }
        // dQ = lower(dO V^T) K + dO S^T: the forward walk over (dO, V, K), its states V^T K = S^T
        fla::WalkParams w{};
        w.q = go.ptr, w.k = v.ptr, w.v = k.ptr, w.o = const_cast<void *>(dq.ptr);
        w.qs_b = go.strides[0], w.qs_h = go.strides[1], w.qs_n = go.strides[2];
        w.ks_b = v.strides[0], w.ks_h = v.strides[1], w.ks_n = v.strides[2];
        w.vs_b = k.strides[0], w.vs_h = k.strides[1], w.vs_n = k.strides[2];
        w.os_b = dq.strides[0], w.os_h = dq.strides[1], w.os_n = dq.strides[2];
        w.H = (int32_t)H, w.N = (int32_t)N, w.BH = (int32_t)(B * H), w.wqk = (int32_t)dv, w.wv = (int32_t)dqk;
        w.n_chunks = (int32_t)wp.n_chunks, w.seg_chunks = (int32_t)wp.seg_chunks, w.n_seg = (int32_t)wp.n_seg;
        w.init = wp.n_seg > 1 ? static_cast<const float *>(state_in) : nullptr, w.init_transposed = 1;
        if (fmap) {  // q holds phi(xq): dQ leaves multiplied by the slope computed from it
            w.fmap = fmap, w.slope_y = q.ptr;
            w.sy_b = q.strides[0], w.sy_h = q.strides[1], w.sy_n = q.strides[2];
        }
        if (nx) w.dn = nx->dn, w.zc = zc, nx->fused = true;  // dQ's term of the normaliser inside its walk
        if (fla::walk_fwd(dtype, wp.D, w, s) != hipSuccess) return FLA_ERR_LAUNCH;
        // dV, dK: the reverse walk over the same segments
        fla::WalkParams r{};
        r.q = q.ptr, r.k = k.ptr, r.v = v.ptr, r.go = go.ptr;
        r.dk = const_cast<void *>(dk.ptr), r.dv = const_cast<void *>(dvv.ptr);
        r.qs_b = q.strides[0], r.qs_h = q.strides[1], r.qs_n = q.strides[2];
        r.ks_b = k.strides[0], r.ks_h = k.strides[1], r.ks_n = k.strides[2];
        r.vs_b = v.strides[0], r.vs_h = v.strides[1], r.vs_n = v.strides[2];
        r.gs_b = go.strides[0], r.gs_h = go.strides[1], r.gs_n = go.strides[2];
        r.dks_b = dk.strides[0], r.dks_h = dk.strides[1], r.dks_n = dk.strides[2];
        r.dvs_b = dvv.strides[0], r.dvs_h = dvv.strides[1], r.dvs_n = dvv.strides[2];
        r.H = (int32_t)H, r.N = (int32_t)N, r.BH = (int32_t)(B * H), r.wqk = (int32_t)dqk, r.wv = (int32_t)dv;
        r.n_chunks = (int32_t)wp.n_chunks, r.seg_chunks = (int32_t)wp.seg_chunks, r.n_seg = (int32_t)wp.n_seg;
        r.init = entry, r.fmap = fmap;  // (dK: the slope from phi(xk) in the K tile)
        if (nx) r.dn = nx->dn, r.rc = rcv;  // dK's terms
        return fla::walk_dkdv(dtype, wp.D, r, s) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
    }
    if (walk) {  // (the states forward saved are per 128-row chunk: only this path reads them)
        if (wp.n_seg > 1 &&
            (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < wp.work_bytes))
            return FLA_ERR_WORKSPACE;
        if (reinterpret_cast<uintptr_t>(state_in) % 16 != 0) return FLA_ERR_WORKSPACE;
        hipStream_t s = static_cast<hipStream_t>(stream);
        const float *entry = nullptr;
        if (wp.n_seg > 1)
            if (int rc = walk_entry_states(wp, q, go, B, H, N, dqk, dv, dtype, 1, workspace, nullptr, &entry, s)) return rc;
        fla::WalkParams w{};
        w.fmap = fmap;  // q, k hold phi(x): the slopes come from the LDS tiles
        w.q = q.ptr, w.k = k.ptr, w.v = v.ptr, w.go = go.ptr;
        w.dq = const_cast<void *>(dq.ptr), w.dk = const_cast<void *>(dk.ptr), w.dv = const_cast<void *>(dvv.ptr);
        w.qs_b = q.strides[0], w.qs_h = q.strides[1], w.qs_n = q.strides[2];
        w.ks_b = k.strides[0], w.ks_h = k.strides[1], w.ks_n = k.strides[2];
        w.vs_b = v.strides[0], w.vs_h = v.strides[1], w.vs_n = v.strides[2];
        w.gs_b = go.strides[0], w.gs_h = go.strides[1], w.gs_n = go.strides[2];
        w.dqs_b = dq.strides[0], w.dqs_h = dq.strides[1], w.dqs_n = dq.strides[2];
        w.dks_b = dk.strides[0], w.dks_h = dk.strides[1], w.dks_n = dk.strides[2];
        w.dvs_b = dvv.strides[0], w.dvs_h = dvv.strides[1], w.dvs_n = dvv.strides[2];
        w.H = (int32_t)H, w.N = (int32_t)N, w.BH = (int32_t)(B * H), w.wqk = (int32_t)dqk, w.wv = (int32_t)dv;
        w.n_chunks = (int32_t)wp.n_chunks, w.seg_chunks = (int32_t)wp.seg_chunks, w.n_seg = (int32_t)wp.n_seg;
        w.init = entry;
        if (nx) {
            w.saved = const_cast<void *>(state_in);
        } else {  // forward's entry states and, behind them, its state after the last chunk
            w.xinit = static_cast<const float *>(state_in);
            w.xtotal = reinterpret_cast<const float *>(static_cast<const char *>(state_in) + wp.entry_bytes);
        }
        if (nx) {
            const int64_t vb = walk_vec_bytes(B, H, N, dqk, dv);
            float *zc = static_cast<float *>(nx->vec), *rcv = reinterpret_cast<float *>(static_cast<char *>(nx->vec) + vb);
            if (zc_saved) zc = const_cast<float *>(zc_saved);
            else if (int rc = walk_chunk_vectors(wp, k, dqk, nullptr, 0, zc, B, H, N, dtype, s)) return rc;
            if (int rc = walk_chunk_vectors(wp, q, dqk, nx->dn, 1, rcv, B, H, N, dtype, s)) return rc;
            w.dn = nx->dn, w.zc = zc, w.rc = rcv;
            nx->fused = true;
        }
        return fla::walk_bwd(dtype, wp.D, w, s) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
    }
    if (wp.ok) state_in = nullptr;  // not in the 256-row chunks' format: recomputed below
    if (fmap_late) set_output_slope(pq, fmap, q), set_output_slope(pk, fmap, k);
    const int64_t sb = shared_state_bytes(B, H, N, dqk, dv);
    if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < sb * (state_in ? 3 : 4))
        return FLA_ERR_WORKSPACE;
    float *w = static_cast<float *>(workspace);
    void *state_v = static_cast<char *>(workspace) + 2 * sb;
    const void *state_f = state_in;
    if (!state_f) {
        void *mine = static_cast<char *>(workspace) + 3 * sb;
        if (int rc = chunk_states(k, v, B, H, N, dqk, dv, 0, dtype, w, mine, stream)) return rc;
        state_f = mine;
    }
    if (int rc = chunk_states(q, go, B, H, N, dqk, dv, 1, dtype, w, state_v, stream)) return rc;
    // One launch for the three products: a workgroup evaluates dQ, dV and dK of its chunk in turn,
    // so q, k, v and dO come from memory once.  dQ reads the forward state [D_v][D_qk] as its own
    // [D_c = D_v][D_o = D_qk] transposed state; dK reads the state of dV transposed.
    fla::TriBatch b;
    b.p[0] = pq, b.p[0].state = state_f, b.p[0].state_transposed = 1;
    b.p[1] = pv, b.p[1].state = state_v, b.p[1].state_transposed = 0;
    b.p[2] = pk, b.p[2].state = state_v, b.p[2].state_transposed = 1;
    return lookup_chunked_batch(dtype, dqk)(b, 3, static_cast<hipStream_t>(stream)) == hipSuccess ? FLA_OK
                                                                                                   : FLA_ERR_LAUNCH;
}

// O = tril(phi(xq) phi(xk)^T) v with mapped = {phi(xq), phi(xk)} as further outputs.  Chunk-wise
// (chunked != 0): the kernels map on load where they can (the state kernel xk, the main kernel its
// rows of xq); any other shape or layout, and the quadratic kernels, get one element-wise pass
// per operand and then the plain operator on phi(xq), phi(xk).
int feature_forward(const View &vxq, const View &vxk, const View &vv, const View &vo, const View (&mapped)[2], int64_t B,
                    int64_t H, int64_t N, int64_t dqk, int64_t dv, int fmap, int dtype, int chunked, void *state_out,
                    int32_t *state_valid, void *workspace, int64_t workspace_bytes, void *stream,
                    WalkNorm *nx = nullptr) {
    const View all[] = {vxq, vxk, vv, vo, mapped[0], mapped[1]};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    {
        const Span ins[] = {span_of(vxq, B, H, N, dqk), span_of(vxk, B, H, N, dqk), span_of(vv, B, H, N, dv)};
        const Span outs[] = {span_of(vo, B, H, N, dv), span_of(mapped[0], B, H, N, dqk), span_of(mapped[1], B, H, N, dqk)};
        if (int rc = check_alias(ins, 3, outs, 3)) return rc;
    }
    if (chunked) {
        bool done = false;
        if (int rc = chunked_forward(vxq, vxk, vv, vo, B, H, N, dqk, dv, dtype, state_out, state_valid, workspace,
                                     workspace_bytes, stream, fmap, mapped, &done, nx))
            return rc;
        if (done) return FLA_OK;
    }
    if (int rc = launch_feature_pass(1, fmap, vxq, mapped[0], B, H, N, dqk, dtype, stream)) return rc;
    if (int rc = launch_feature_pass(1, fmap, vxk, mapped[1], B, H, N, dqk, dtype, stream)) return rc;
    if (!chunked) return run_tri(mapped[0], mapped[1], vv, vo, B, H, N, dqk, dv, 0, dtype, stream);
    return chunked_forward(mapped[0], mapped[1], vv, vo, B, H, N, dqk, dv, dtype, state_out, state_valid, workspace,
                           workspace_bytes, stream, 0, nullptr, nullptr, nx);
}

int forward(const View &q, const View &k, const View &v, const View &o, int64_t B, int64_t H, int64_t N,
            int64_t dqk, int64_t dv, int dtype, void *stream) {
    const View all[] = {q, k, v, o};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (int rc = check_alias_fwd(q, k, v, o, B, H, N, dqk, dv)) return rc;
    return run_tri(q, k, v, o, B, H, N, dqk, dv, 0, dtype, stream);
}

// The three gradient products for validated views.
int backward_products(const View &go, const View &q, const View &k, const View &v, const View &dq, const View &dk,
                      const View &dv, int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dvw, int dtype,
                      void *stream) {
    // dQ = lower(dO V^T) K ; dV = upper(K Q^T) dO ; dK = upper(V dO^T) Q
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    // Equal padded widths up to 128: all three products run the same kernel, so they go out as
    // one launch (workgroups of the next product fill the previous one's tail).
    if (pad_index(dqk) == pad_index(dvw) && padded(dqk) <= 128) {
        fla::TriBatch b;
        b.p[0] = make_params(go, v, k, dq, B, H, N, dvw, dqk, 0);
        b.p[1] = make_params(k, q, go, dv, B, H, N, dqk, dvw, 1);
        b.p[2] = make_params(v, go, q, dk, B, H, N, dvw, dqk, 1);
        if (fla::fast_path_ok(b.p[0]) && fla::fast_path_ok(b.p[1]) && fla::fast_path_ok(b.p[2])) {
            const hipError_t e = lookup_batch(dtype, dqk)(b, 3, static_cast<hipStream_t>(stream));
            if (e == hipSuccess) return FLA_OK;
            if (e != hipErrorNotSupported) return FLA_ERR_LAUNCH;
        }
    }
    if (int rc = run_tri(go, v, k, dq, B, H, N, dvw, dqk, 0, dtype, stream)) return rc;
    if (int rc = run_tri(k, q, go, dv, B, H, N, dqk, dvw, 1, dtype, stream)) return rc;
    return run_tri(v, go, q, dk, B, H, N, dvw, dqk, 1, dtype, stream);
}

// The same gradients with dV and dK from one stream of (Q, dO) tiles (fla_tri_pair.h) and dQ as a
// product of its own: equal padded head dims up to 128, operands on the fast path.
int backward_fused_dkdv(const View &go, const View &q, const View &k, const View &v, const View &dq, const View &dk,
                        const View &dv, int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dvw, int dtype,
                        void *stream) {
    const View all[] = {go, q, k, v, dq, dk, dv};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (int rc = check_alias_bwd(go, q, k, v, nullptr, dq, dk, dv, B, H, N, dqk, dvw)) return rc;
    if (pad_index(dqk) != pad_index(dvw) || padded(dqk) > 128) return FLA_ERR_UNSUPPORTED;
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    const TriParams pq = make_params(go, v, k, dq, B, H, N, dvw, dqk, 0);
    const TriParams pv = make_params(k, q, go, dv, B, H, N, dqk, dvw, 1);
    const TriParams pk = make_params(v, go, q, dk, B, H, N, dvw, dqk, 1);
    if (!fla::fast_path_ok(pq) || !fla::fast_path_ok(pv) || !fla::fast_path_ok(pk)) return FLA_ERR_UNSUPPORTED;
    typedef hipError_t (*pair_fn)(const TriParams &, const TriParams &, hipStream_t);
    static const pair_fn table[3][2] = {{fla::FLA_PAIR_NAME(0, 32), fla::FLA_PAIR_NAME(1, 32)},
                                        {fla::FLA_PAIR_NAME(0, 64), fla::FLA_PAIR_NAME(1, 64)},
                                        {fla::FLA_PAIR_NAME(0, 128), fla::FLA_PAIR_NAME(1, 128)}};
    if (table[pad_index(dqk)][dtype](pv, pk, static_cast<hipStream_t>(stream)) != hipSuccess) return FLA_ERR_LAUNCH;
    return run_tri(go, v, k, dq, B, H, N, dvw, dqk, 0, dtype, stream);
}

int backward(const View &go, const View &q, const View &k, const View &v, const View &dq, const View &dk,
             const View &dv, int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dvw, int dtype, void *stream) {
    const View all[] = {go, q, k, v, dq, dk, dv};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (int rc = check_alias_bwd(go, q, k, v, nullptr, dq, dk, dv, B, H, N, dqk, dvw)) return rc;
    return backward_products(go, q, k, v, dq, dk, dv, B, H, N, dqk, dvw, dtype, stream);
}

// ---- normalised linear attention: out = tril(Q K^T) V / (q . cumsum(k) + eps)

struct NormLayout {
    int lpr;
    int64_t chunks, sums_bytes, do_bytes, dn_bytes;
    int64_t vec_bytes;    // chunk-wise walk kernels: one set of per-chunk running vectors (two are kept)
    int64_t norm_bytes;   // the normaliser's own scratch: dO, dn, two sets of chunk sums, two sets of vectors
    int64_t chunk_bytes;  // behind it: scratch of the chunk-wise product evaluation (0 when quadratic)
};

NormLayout norm_layout(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv, int chunked) {
    NormLayout l;
    l.lpr = fla::norm_lanes_per_row((int)(dqk > dv ? dqk : dv));
    const int64_t rows = fla::norm_chunk_rows(l.lpr);
    l.chunks = (N + rows - 1) / rows;
    l.sums_bytes = B * H * l.chunks * (l.lpr * 8) * 4;
    l.do_bytes = (B * H * N * dv * 2 + 15) / 16 * 16;
    l.dn_bytes = (B * H * N * 4 + 15) / 16 * 16;
    l.sums_bytes = (l.sums_bytes + 15) / 16 * 16;
    l.vec_bytes = chunked ? walk_vec_bytes(B, H, N, dqk, dv) : 0;
    l.norm_bytes = l.do_bytes + l.dn_bytes + 2 * l.sums_bytes + 2 * l.vec_bytes;
    l.chunk_bytes = chunked ? chunked_op_workspace_bytes(B, H, N, dqk, dv) : 0;
    return l;
}

void norm_common(fla::NormParams &p, const View &q, const View &k, int64_t B, int64_t H, int64_t N, int64_t dqk,
                 int64_t dv, const NormLayout &l) {
    p = fla::NormParams{};
    p.q = q.ptr, p.k = k.ptr;
    p.qs_b = q.strides[0], p.qs_h = q.strides[1], p.qs_n = q.strides[2];
    p.ks_b = k.strides[0], p.ks_h = k.strides[1], p.ks_n = k.strides[2];
    p.H = (int32_t)H, p.N = (int32_t)N, p.BH = (int32_t)(B * H), p.dqk = (int32_t)dqk, p.dv = (int32_t)dv;
    p.n_chunks = (int32_t)l.chunks;
    p.vec_q = vec_ok(q, dqk), p.vec_k = vec_ok(k, dqk);
}

hipError_t norm_launch(int which, int dtype, int lpr, const fla::NormParams &p, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the operands this pass touches all allow 16-byte accesses?
    const bool vec = which == 0   ? (p.vec_q && p.vec_k && p.vec_a && p.vec_out)
                     : which == 1 ? (p.vec_a && p.vec_b && p.vec_out)
                                  : (p.vec_q && p.vec_k && p.vec_dq && p.vec_dk);
    return dtype == FLA_DTYPE_BF16 ? fla::launch_norm<__bf16>(which, lpr, vec, p, s)
                                   : fla::launch_norm<_Float16>(which, lpr, vec, p, s);
}

int check_norm_args(int64_t B, int64_t H, int64_t N, int64_t dqk, int64_t dv, int dtype) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (dqk < 1 || dqk > 256) return FLA_ERR_HEAD_DIM;
    if (dv < 1 || dv > 256) return FLA_ERR_V_HEAD_DIM;
    // the grid's second dimension is the (batch, head) index
    if (B * H > 65535) return FLA_ERR_SHAPE;
    return FLA_OK;
}

// Forward with the normaliser inside the product kernel: the row sums of the masked scores are
// the normaliser (q_i . sum_{j<=i} k_j = sum_j q_i . k_j), so the fast kernel divides before it
// stores and no extra pass runs.  Returns 1 when this shape / layout has no such kernel (the
// caller then normalises with the separate passes), 0 on success, a negative code on failure.
int fused_normalised_forward(const View &q, const View &k, const View &v, const View &o, float *denom, int64_t B,
                             int64_t H, int64_t N, int64_t dqk, int64_t dv, float eps, int dtype, void *stream) {
    const bool split = dv > 128 && (dqk <= 64 || dqk > 128);
    const int64_t w0 = split ? 128 : dv;
    TriParams p0 = make_params(q, k, v, o, B, H, N, dqk, w0, 0);
    if (chunk_rows(dqk, w0) == 0 || !fla::fast_path_ok(p0)) return 1;
    p0.denom = denom, p0.eps = eps;
    if (!split) return lookup(dtype, dqk, w0)(p0, static_cast<hipStream_t>(stream)) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
    const View v_hi{static_cast<const char *>(v.ptr) + 128 * 2, v.strides};
    const View o_hi{static_cast<const char *>(o.ptr) + 128 * 2, o.strides};
    TriParams p1 = make_params(q, k, v_hi, o_hi, B, H, N, dqk, dv - 128, 0);
    if (chunk_rows(dqk, dv - 128) == 0 || !fla::fast_path_ok(p1)) return 1;
    p1.denom = denom, p1.eps = eps;  // both halves see the same scores and write the same n
    if (lookup(dtype, dqk, w0)(p0, static_cast<hipStream_t>(stream)) != hipSuccess) return FLA_ERR_LAUNCH;
    return lookup(dtype, dqk, dv - 128)(p1, static_cast<hipStream_t>(stream)) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
}

// fmap != 0: q0, k0 hold the arguments xq, xk of the feature map and mapped = {phi(xq), phi(xk)} are
// further outputs; the normaliser is that of phi(xq), phi(xk).
int normalised_forward(const View &q0, const View &k0, const View &v, const View &o, float *denom, int64_t B, int64_t H,
                       int64_t N, int64_t dqk, int64_t dv, float eps, int dtype, int chunked, void *workspace,
                       int64_t workspace_bytes, void *stream, int fmap = 0, const View *mapped = nullptr,
                       void *state_out = nullptr, int32_t *state_valid = nullptr) {
    if (state_valid) *state_valid = 0;
    const View all[] = {q0, k0, v, o};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (!denom) return FLA_ERR_NULL_POINTER;
    if (int rc = check_alias_fwd(q0, k0, v, o, B, H, N, dqk, dv)) return rc;
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    const NormLayout l = norm_layout(B, H, N, dqk, dv, chunked);
    if ((l.chunks > 1 || l.chunk_bytes > 0) &&
        (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < l.norm_bytes + l.chunk_bytes))
        return FLA_ERR_WORKSPACE;
    if (fmap && !chunked) {
        // quadratic product: phi by element-wise passes, then the operator on phi(xq), phi(xk)
        for (int i = 0; i < 2; ++i)
            if (int rc = check_view(mapped[i])) return rc;
        if (int rc = launch_feature_pass(1, fmap, q0, mapped[0], B, H, N, dqk, dtype, stream)) return rc;
        if (int rc = launch_feature_pass(1, fmap, k0, mapped[1], B, H, N, dqk, dtype, stream)) return rc;
        return normalised_forward(mapped[0], mapped[1], v, o, denom, B, H, N, dqk, dv, eps, dtype, 0, workspace,
                                  workspace_bytes, stream);
    }
    // chunk-wise walk kernels compute n and divide by it themselves
    WalkNorm nx{denom, eps, nullptr,
                workspace ? static_cast<char *>(workspace) + l.do_bytes + l.dn_bytes + 2 * l.sums_bytes : nullptr, false, false};
    const View &q = fmap ? mapped[0] : q0, &k = fmap ? mapped[1] : k0;
    if (!chunked) {
        const int rc = fused_normalised_forward(q, k, v, o, denom, B, H, N, dqk, dv, eps, dtype, stream);
        if (rc <= 0) return rc;
    }
    if (fmap) {
        const View both[2] = {mapped[0], mapped[1]};
        if (int rc = feature_forward(q0, k0, v, o, both, B, H, N, dqk, dv, fmap, dtype, 1, state_out, state_valid,
                                     static_cast<char *>(workspace) + l.norm_bytes, l.chunk_bytes, stream, &nx))
            return rc;
        if (nx.fused) return FLA_OK;
    } else if (chunked) {
        if (int rc = chunked_forward(q, k, v, o, B, H, N, dqk, dv, dtype, state_out, state_valid,
                                     static_cast<char *>(workspace) + l.norm_bytes, l.chunk_bytes, stream, 0, nullptr,
                                     nullptr, &nx))
            return rc;
        if (nx.fused) return FLA_OK;
    } else if (int rc = run_tri(q, k, v, o, B, H, N, dqk, dv, 0, dtype, stream)) {
        return rc;
    }
    fla::NormParams p;
    norm_common(p, q, k, B, H, N, dqk, dv, l);
    p.a = o.ptr, p.out = const_cast<void *>(o.ptr);  // normalised in place
    p.as_b = p.os_b = o.strides[0], p.as_h = p.os_h = o.strides[1], p.as_n = p.os_n = o.strides[2];
    p.vec_a = p.vec_out = vec_ok(o, dv);
    p.denom = denom;
    p.ksum = static_cast<float *>(workspace);
    p.eps = eps;
    return norm_launch(0, dtype, l.lpr, p, stream) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
}

int normalised_backward(const View &go, const View &q, const View &k, const View &v, const View &o,
                        const float *denom, const View &dq, const View &dk, const View &dvv, int64_t B, int64_t H,
                        int64_t N, int64_t dqk, int64_t dv, int dtype, int chunked, void *workspace,
                        int64_t workspace_bytes, void *stream, int fmap = 0, const void *state_in = nullptr) {
    // fmap != 0: q, k hold phi(xq), phi(xk) and dq, dk leave as gradients with respect to xq, xk (the
    // slope is multiplied in by the last pass, after the normaliser's own terms have been added)
    const View all[] = {go, q, k, v, o, dq, dk, dvv};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (!denom) return FLA_ERR_NULL_POINTER;
    if (int rc = check_alias_bwd(go, q, k, v, &o, dq, dk, dvv, B, H, N, dqk, dv)) return rc;
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    const NormLayout l = norm_layout(B, H, N, dqk, dv, chunked);
    if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 || workspace_bytes < l.norm_bytes + l.chunk_bytes)
        return FLA_ERR_WORKSPACE;
    char *ws = static_cast<char *>(workspace);
    void *dO = ws;
    float *dn = reinterpret_cast<float *>(ws + l.do_bytes);
    float *ksum = reinterpret_cast<float *>(ws + l.do_bytes + l.dn_bytes);
    float *wsum = reinterpret_cast<float *>(ws + l.do_bytes + l.dn_bytes + l.sums_bytes);
    const int64_t do_strides[4] = {H * N * dv, N * dv, dv, 1};
    const View dOv{dO, do_strides};

    fla::NormParams p;
    norm_common(p, q, k, B, H, N, dqk, dv, l);
    p.denom = const_cast<float *>(denom), p.dn = dn, p.ksum = ksum, p.wsum = wsum;
    // dO = g / n, dn = -(g . out) / n
    p.a = go.ptr, p.as_b = go.strides[0], p.as_h = go.strides[1], p.as_n = go.strides[2], p.vec_a = vec_ok(go, dv);
    p.b = o.ptr, p.bs_b = o.strides[0], p.bs_h = o.strides[1], p.bs_n = o.strides[2], p.vec_b = vec_ok(o, dv);
    p.out = dO, p.os_b = do_strides[0], p.os_h = do_strides[1], p.os_n = do_strides[2], p.vec_out = vec_ok(dOv, dv);
    if (norm_launch(1, dtype, l.lpr, p, stream) != hipSuccess) return FLA_ERR_LAUNCH;
    // gradients of the unnormalised product
    WalkNorm nx{nullptr, 0.f, dn, ws + l.do_bytes + l.dn_bytes + 2 * l.sums_bytes, false, false};
    if (chunked) {
        // the walk kernels add the normaliser's terms (and apply the slope of a feature map) themselves
        if (int rc = chunked_backward(dOv, q, k, v, dq, dk, dvv, B, H, N, dqk, dv, dtype, state_in, ws + l.norm_bytes,
                                      l.chunk_bytes, stream, fmap, &nx))
            return rc;
        if (nx.fused && !nx.dk_pending) return FLA_OK;
    } else if (int rc = backward_products(dOv, q, k, v, dq, dk, dvv, B, H, N, dqk, dv, dtype, stream)) {
        return rc;
    }
    // the normaliser's own terms
    p.dq = const_cast<void *>(dq.ptr), p.dqs_b = dq.strides[0], p.dqs_h = dq.strides[1], p.dqs_n = dq.strides[2];
    p.dk = const_cast<void *>(dk.ptr), p.dks_b = dk.strides[0], p.dks_h = dk.strides[1], p.dks_n = dk.strides[2];
    p.vec_dq = vec_ok(dq, dqk), p.vec_dk = vec_ok(dk, dqk);
    p.fmap = fmap;
    p.only_dk = nx.fused && nx.dk_pending;  // (dq is complete, slope included)
    return norm_launch(2, dtype, l.lpr, p, stream) == hipSuccess ? FLA_OK : FLA_ERR_LAUNCH;
}

// ---- polynomial score map: out = lower(f(Xq Xk^T)) V, f(u) = c0 + c1 u + c2 u^2

// [a | x] side by side, 8 elements per thread: columns [0, split) hold a (zero beyond its width),
// columns [split, split + rp) hold x (zero beyond its width); out is contiguous (B, H, N, split + rp).
// bias_mode 1 / 2 puts one more value right after a, in column wa: bias[row] / the constant 1.
template <typename T>
__global__ __launch_bounds__(256) void pack_pair_kernel(const T *a, int64_t as_b, int64_t as_h, int64_t as_n, int wa,
                                                        const T *x, int64_t xs_b, int64_t xs_h, int64_t xs_n, int wx,
                                                        T *out, int H, int64_t N, int split, int rp, int64_t total,
                                                        int bias_mode, const float *bias) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    const int cpr = (split + rp) / 8;  // 8-element chunks per row
    const int64_t row = t / cpr;
    const int c8 = (int)(t - row * cpr) * 8;
    const int64_t bh = row / N, n = row - bh * N;
    const int64_t b = bh / H, h = bh - b * H;
    fla::u32x4 w = {0u, 0u, 0u, 0u};
    if (c8 < split) {
        if (c8 < wa) {
            w = *reinterpret_cast<const fla::u32x4 *>(a + b * as_b + h * as_h + n * as_n + c8);
        } else if (c8 == wa && bias_mode) {
            const T one = static_cast<T>(bias_mode == 1 ? bias[row] : 1.0f);
            w[0] = (uint32_t)__builtin_bit_cast(unsigned short, one);
        }
    } else if (c8 - split < wx) {
        w = *reinterpret_cast<const fla::u32x4 *>(x + b * xs_b + h * xs_h + n * xs_n + (c8 - split));
    }
    *reinterpret_cast<fla::u32x4 *>(out + row * (split + rp) + c8) = w;
}

template <typename T>
hipError_t launch_pack(const View &a, int wa, const View &x, int wx, void *out, int64_t B, int64_t H, int64_t N, int split,
                 int rp, int bias_mode, const float *bias, hipStream_t s) {
    const int64_t total = B * H * N * ((split + rp) / 8);
    return fla::launch_kernel<pack_pair_kernel<T>>(dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                              static_cast<const T *>(a.ptr), a.strides[0], a.strides[1], a.strides[2], wa,
                              static_cast<const T *>(x.ptr), x.strides[0], x.strides[1], x.strides[2], wx,
                              static_cast<T *>(out), (int)H, N, split, rp, total, bias_mode, bias);
}

struct PolyLayout {
    int64_t split, rp, width, packed_bytes;
    int mode;  // TriParams::poly_on of the dual-score products: 2 (half layout) or 3 (tail layout)
    // normalised backward: dO = g / n and dn, then the packed operands
    int64_t do_bytes, dn_bytes;
};

// split: where the second operand starts; rp: r rounded up to whole 16-byte chunks.  Without the
// bias column the first operand is padded to half of the contraction the dual-score kernel is built
// for (the kernel skips the empty chunks); with it (normalised backward) D_v + 1 columns are needed,
// and when those do not fit the half the second operand goes to the last 32 columns instead.
PolyLayout poly_layout(int64_t B, int64_t H, int64_t N, int64_t r, int64_t dv, int with_bias) {
    PolyLayout l;
    const int64_t need = dv + (with_bias ? 8 : 0);  // the bias takes a 16-byte chunk of its own
    const int64_t half = need <= 32 ? 32 : need <= 64 ? 64 : need <= 128 ? 128 : 0;
    const int64_t dc_tail = need + 32 <= 64 ? 64 : need + 32 <= 128 ? 128 : 256;
    if (half != 0 && 2 * half <= dc_tail) {
        l.split = half, l.mode = 2;
    } else {
        l.split = dc_tail - 32, l.mode = 3;
    }
    l.rp = l.mode == 3 ? 32 : (r + 7) / 8 * 8;
    l.width = l.split + l.rp;
    l.packed_bytes = (B * H * N * l.width * 2 + 15) / 16 * 16;
    l.do_bytes = with_bias ? (B * H * N * dv * 2 + 15) / 16 * 16 : 0;
    l.dn_bytes = with_bias ? (B * H * N * 4 + 15) / 16 * 16 : 0;
    return l;
}

int check_poly_args(int64_t B, int64_t H, int64_t N, int64_t r, int64_t dv, int dtype, const float *coef) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (!coef) return FLA_ERR_NULL_POINTER;
    if (r < 1 || r > 32) return FLA_ERR_HEAD_DIM;
    if (dv < 1 || dv > 128) return FLA_ERR_V_HEAD_DIM;
    return FLA_OK;
}

// every product of this operator exists only as a fast-path kernel
bool poly_ok(const TriParams &p, int64_t dc, int64_t dout) { return chunk_rows(dc, dout) != 0 && fla::fast_path_ok(p); }

int launch_poly(TriParams p, int64_t dc, int64_t dout, int dtype, int mode, float c0, float c1, float c2, void *stream) {
    p.poly[0] = c0, p.poly[1] = c1, p.poly[2] = c2, p.poly_on = mode;
    const hipError_t e = lookup(dtype, dc, dout)(p, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? FLA_OK : e == hipErrorNotSupported ? FLA_ERR_UNSUPPORTED : FLA_ERR_LAUNCH;
}

int poly_forward(const View &xq, const View &xk, const View &v, const View &o, float *denom, int64_t B, int64_t H,
                 int64_t N, int64_t r, int64_t dv, const float *coef, float eps, int dtype, void *stream) {
    const View all[] = {xq, xk, v, o};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (int rc = check_alias_fwd(xq, xk, v, o, B, H, N, r, dv)) return rc;
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    if (denom && B * H > 65535) return FLA_ERR_SHAPE;
    TriParams p = make_params(xq, xk, v, o, B, H, N, r, dv, 0);
    if (!poly_ok(p, r, dv)) return FLA_ERR_UNSUPPORTED;
    p.denom = denom, p.eps = eps;
    return launch_poly(p, r, dv, dtype, 1, coef[0], coef[1], coef[2], stream);
}

int poly_backward(const View &go, const View &xq, const View &xk, const View &v, const View *o, const float *denom,
                  const View &dxq, const View &dxk, const View &dvv, int64_t B, int64_t H, int64_t N, int64_t r,
                  int64_t dv, const float *coef, int dtype, void *workspace, int64_t workspace_bytes, void *stream) {
    const View all[] = {go, xq, xk, v, dxq, dxk, dvv};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    const bool normalised = o != nullptr;
    if (normalised) {
        if (int rc = check_view(*o)) return rc;
        if (!denom) return FLA_ERR_NULL_POINTER;
        if (B * H > 65535) return FLA_ERR_SHAPE;
    }
    if (int rc = check_alias_bwd(go, xq, xk, v, o, dxq, dxk, dvv, B, H, N, r, dv)) return rc;
    if (B == 0 || H == 0 || N == 0) return FLA_OK;
    const PolyLayout l = poly_layout(B, H, N, r, dv, normalised);
    if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 16 != 0 ||
        workspace_bytes < 2 * l.packed_bytes + l.do_bytes + l.dn_bytes)
        return FLA_ERR_WORKSPACE;
    // the packing kernel and the products below use 16-byte accesses throughout
    if (!(vec_ok(go, dv) && vec_ok(v, dv) && vec_ok(xq, r) && vec_ok(xk, r) && vec_ok(dxq, r) && vec_ok(dxk, r) &&
          vec_ok(dvv, dv)))
        return FLA_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    char *ws = static_cast<char *>(workspace);
    void *p1 = ws, *p2 = ws + l.packed_bytes;  // [dO (| dn) | xq], [V (| 1) | xk]
    void *dO = ws + 2 * l.packed_bytes;
    float *dn = reinterpret_cast<float *>(ws + 2 * l.packed_bytes + l.do_bytes);
    const int64_t do_strides[4] = {H * N * dv, N * dv, dv, 1};
    View g = go;
    if (normalised) {
        // out = O / n: dO = g / n, dn = -(g . out) / n; the dn term enters u1 as a bias column
        const int lpr = fla::norm_lanes_per_row((int)dv);
        fla::NormParams np{};
        np.H = (int32_t)H, np.N = (int32_t)N, np.BH = (int32_t)(B * H), np.dqk = (int32_t)dv, np.dv = (int32_t)dv;
        const int64_t rows = fla::norm_chunk_rows(lpr);
        np.n_chunks = (int32_t)((N + rows - 1) / rows);
        np.denom = const_cast<float *>(denom), np.dn = dn;
        np.a = go.ptr, np.as_b = go.strides[0], np.as_h = go.strides[1], np.as_n = go.strides[2], np.vec_a = vec_ok(go, dv);
        np.b = o->ptr, np.bs_b = o->strides[0], np.bs_h = o->strides[1], np.bs_n = o->strides[2], np.vec_b = vec_ok(*o, dv);
        np.out = dO, np.os_b = do_strides[0], np.os_h = do_strides[1], np.os_n = do_strides[2], np.vec_out = 1;
        if (norm_launch(1, dtype, lpr, np, stream) != hipSuccess) return FLA_ERR_LAUNCH;
        g = View{dO, do_strides};
    }
    const int bias1 = normalised ? 1 : 0, bias2 = normalised ? 2 : 0;
    const auto pack = dtype == FLA_DTYPE_BF16 ? launch_pack<__bf16> : launch_pack<_Float16>;
    if (pack(g, (int)dv, xq, (int)r, p1, B, H, N, (int)l.split, (int)l.rp, bias1, dn, s) != hipSuccess) return FLA_ERR_LAUNCH;
    if (pack(v, (int)dv, xk, (int)r, p2, B, H, N, (int)l.split, (int)l.rp, bias2, nullptr, s) != hipSuccess)
        return FLA_ERR_LAUNCH;
    const int64_t ps[4] = {H * N * l.width, N * l.width, l.width, 1};
    const View P1{p1, ps}, P2{p2, ps};
    // dV = upper(f(Xk Xq^T)) dO
    const TriParams pv = make_params(xk, xq, g, dvv, B, H, N, r, dv, 1);
    // dXq = lower((dO V^T + dn 1^T) f'(Xq Xk^T)) Xk, dXk = upper((V dO^T + 1 dn^T) f'(Xk Xq^T)) Xq; f'(u) = c1 + 2 c2 u
    const TriParams pq = make_params(P1, P2, xk, dxq, B, H, N, l.width, r, 0);
    const TriParams pk = make_params(P2, P1, xq, dxk, B, H, N, l.width, r, 1);
    if (!poly_ok(pv, r, dv) || !poly_ok(pq, l.width, r) || !poly_ok(pk, l.width, r)) return FLA_ERR_UNSUPPORTED;
    if (int rc = launch_poly(pv, r, dv, dtype, 1, coef[0], coef[1], coef[2], stream)) return rc;
    if (int rc = launch_poly(pq, l.width, r, dtype, l.mode, coef[1], 2.0f * coef[2], 0.f, stream)) return rc;
    return launch_poly(pk, l.width, r, dtype, l.mode, coef[1], 2.0f * coef[2], 0.f, stream);
}

}  // namespace

extern "C" {

int fla_abi_version(void) { return FLA_ABI_VERSION; }

const char *fla_strerror(int status) {
    switch (status) {
        case FLA_OK: return "ok";
        case FLA_ERR_NULL_POINTER: return "a required pointer is NULL";
        case FLA_ERR_DTYPE: return "dtype must be FLA_DTYPE_BF16 or FLA_DTYPE_F16";
        case FLA_ERR_HEAD_DIM: return "Only head_dims <= 256 are supported.";
        case FLA_ERR_V_HEAD_DIM:
            return "value head dimension must be a power of 2 no larger than the padded query/key head dimension";
        case FLA_ERR_SHAPE: return "B, H and N must be non-negative and B*H, N at most 2^30";
        case FLA_ERR_STRIDE: return "strides must be given, non-negative, with innermost stride 1";
        case FLA_ERR_LAUNCH: return "the HIP runtime rejected the kernel launch";
        case FLA_ERR_UNSUPPORTED: return "no kernel was built for this combination";
        case FLA_ERR_WORKSPACE: return "workspace is NULL, not 16-byte aligned, or smaller than fla_chunked_workspace_bytes()";
        case FLA_ERR_ALIAS: return "an output tensor overlaps an input or another output in memory";
        default: return "unknown fla status";
    }
}

int fla_linear_attn_fwd(const void *q, const void *k, const void *v, void *o, int64_t B, int64_t H, int64_t N,
                        int64_t D, const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                        const int64_t *o_strides, int dtype, void *stream) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D < 1 || D > 256) return FLA_ERR_HEAD_DIM;
    return forward({q, q_strides}, {k, k_strides}, {v, v_strides}, {o, o_strides}, B, H, N, D, D, dtype, stream);
}

int fla_linear_attn_bwd(const void *grad_out, const void *q, const void *k, const void *v, void *dq, void *dk,
                        void *dv, int64_t B, int64_t H, int64_t N, int64_t D, const int64_t *go_strides,
                        const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                        const int64_t *dq_strides, const int64_t *dk_strides, const int64_t *dv_strides, int dtype,
                        void *stream) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D < 1 || D > 256) return FLA_ERR_HEAD_DIM;
    return backward({grad_out, go_strides}, {q, q_strides}, {k, k_strides}, {v, v_strides}, {dq, dq_strides},
                    {dk, dk_strides}, {dv, dv_strides}, B, H, N, D, D, dtype, stream);
}

int fla_linear_attn_smallv_fwd(const void *q, const void *k, const void *v, void *o, int64_t B, int64_t H,
                               int64_t N, int64_t D_qk, int64_t D_v, const int64_t *q_strides,
                               const int64_t *k_strides, const int64_t *v_strides, const int64_t *o_strides,
                               int dtype, void *stream) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_qk < 1 || D_qk > 256) return FLA_ERR_HEAD_DIM;
    if (D_v < 1 || next_pow2(D_v) != D_v || D_v > next_pow2(D_qk)) return FLA_ERR_V_HEAD_DIM;
    return forward({q, q_strides}, {k, k_strides}, {v, v_strides}, {o, o_strides}, B, H, N, D_qk, D_v, dtype,
                   stream);
}

int fla_linear_attn_smallv_bwd(const void *grad_out, const void *q, const void *k, const void *v, void *dq,
                               void *dk, void *dv, int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                               const int64_t *go_strides, const int64_t *q_strides, const int64_t *k_strides,
                               const int64_t *v_strides, const int64_t *dq_strides, const int64_t *dk_strides,
                               const int64_t *dv_strides, int dtype, void *stream) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_qk < 1 || D_qk > 256) return FLA_ERR_HEAD_DIM;
    if (D_v < 1 || D_v > 256) return FLA_ERR_V_HEAD_DIM;
    return backward({grad_out, go_strides}, {q, q_strides}, {k, k_strides}, {v, v_strides}, {dq, dq_strides},
                    {dk, dk_strides}, {dv, dv_strides}, B, H, N, D_qk, D_v, dtype, stream);
}

int fla_linear_attn_bwd_fused_dkdv(const void *grad_out, const void *q, const void *k, const void *v, void *dq, void *dk,
                                   void *dv, int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                   const int64_t *go_strides, const int64_t *q_strides, const int64_t *k_strides,
                                   const int64_t *v_strides, const int64_t *dq_strides, const int64_t *dk_strides,
                                   const int64_t *dv_strides, int dtype, void *stream) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_qk < 1 || D_qk > 256) return FLA_ERR_HEAD_DIM;
    if (D_v < 1 || D_v > 256) return FLA_ERR_V_HEAD_DIM;
    return backward_fused_dkdv({grad_out, go_strides}, {q, q_strides}, {k, k_strides}, {v, v_strides}, {dq, dq_strides},
                               {dk, dk_strides}, {dv, dv_strides}, B, H, N, D_qk, D_v, dtype, stream);
}

int fla_tri_xyt_z(const void *x, const void *y, const void *z, void *out, int64_t B, int64_t H, int64_t N,
                  int64_t D_c, int64_t D_o, const int64_t *x_strides, const int64_t *y_strides,
                  const int64_t *z_strides, const int64_t *out_strides, int upper, int dtype, void *stream) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_c < 1 || D_c > 256 || D_o < 1 || D_o > 256) return FLA_ERR_HEAD_DIM;
    const View vx{x, x_strides}, vy{y, y_strides}, vz{z, z_strides}, vo{out, out_strides};
    const View all[] = {vx, vy, vz, vo};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (int rc = check_alias_fwd(vx, vy, vz, vo, B, H, N, D_c, D_o)) return rc;
    return run_tri(vx, vy, vz, vo, B, H, N, D_c, D_o, upper, dtype, stream);
}

int64_t fla_chunked_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t D_c, int64_t D_o) {
    if (B < 0 || H < 0 || N < 0 || D_c < 1 || D_c > 256 || D_o < 1 || D_o > 256) return 0;
    return chunked_bytes(B, H, N, D_c, D_o);
}

int fla_tri_xyt_z_chunked(const void *x, const void *y, const void *z, void *out, int64_t B, int64_t H, int64_t N,
                          int64_t D_c, int64_t D_o, const int64_t *x_strides, const int64_t *y_strides,
                          const int64_t *z_strides, const int64_t *out_strides, int upper, int dtype,
                          void *workspace, int64_t workspace_bytes, void *stream) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_c < 1 || D_c > 256 || D_o < 1 || D_o > 256) return FLA_ERR_HEAD_DIM;
    const View vx{x, x_strides}, vy{y, y_strides}, vz{z, z_strides}, vo{out, out_strides};
    const View all[] = {vx, vy, vz, vo};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    if (int rc = check_alias_fwd(vx, vy, vz, vo, B, H, N, D_c, D_o)) return rc;
    return run_tri_chunked(vx, vy, vz, vo, B, H, N, D_c, D_o, upper, dtype, workspace, workspace_bytes, stream);
}

// Which evaluation of forward + backward is faster on MI355X, from timings of both over grids of
// (head dims, B H, N) (bench.py --crossover): the quadratic kernels' time grows with
// W = B H N^2 D (D: the larger padded head dim), the chunk-wise kernels' with B H N D above a floor
// of launches (four to six for the walk kernels, also for a wide q / k against a narrow v), so each
// of these classes of shapes has one threshold on W.
int fla_linear_attn_prefers_chunked(int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v) {
    if (B < 1 || H < 1 || N < 1 || D_qk < 1 || D_qk > 256 || D_v < 1 || D_v > 256) return 0;
    const double w = (double)B * (double)H * (double)N * (double)N * (double)padded(D_qk > D_v ? D_qk : D_v);
    const WalkPlan wp = walk_plan(B, H, N, D_qk, D_v, true);
    // (padded widths that differ: the quadratic side is the small-V operator, whose wide products are two launches)
    if (wp.ok && pad_index(D_qk) != pad_index(D_v)) return w >= (wp.D <= 64 ? 1e9 : 5e8);
    if (wp.ok) return w >= (wp.D <= 64 ? 4e9 : 8e9);                              // equal padded head dims up to 128
    if (wide_plan(B, H, N, D_qk, D_v).ok) return w >= (D_v <= 64 ? 1e9 : 1.5e10);  // D_qk in (128, 256], D_v <= 128
    if (vsplit_plan(B, H, N, D_qk, D_v).ok) return w >= 3e10;  // D_v in (128, 256] as two column halves of v
    return N >= 4096;  // chunk states in memory, a launch per product and state (measured at 256 / 256)
}

int64_t fla_linear_attn_chunked_state_bytes(int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v) {
    if (B < 0 || H < 0 || N < 0 || D_qk < 1 || D_qk > 256 || D_v < 1 || D_v > 256) return 0;
    return shared_state_bytes(B, H, N, D_qk, D_v);
}

int64_t fla_linear_attn_chunked_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v) {
    if (B < 0 || H < 0 || N < 0 || D_qk < 1 || D_qk > 256 || D_v < 1 || D_v > 256) return 0;
    return chunked_op_workspace_bytes(B, H, N, D_qk, D_v);
}

int fla_linear_attn_chunked_fwd(const void *q, const void *k, const void *v, void *o, int64_t B, int64_t H, int64_t N,
                                int64_t D_qk, int64_t D_v, const int64_t *q_strides, const int64_t *k_strides,
                                const int64_t *v_strides, const int64_t *o_strides, int dtype, void *state_out,
                                int32_t *state_valid, void *workspace, int64_t workspace_bytes, void *stream) {
    if (state_valid) *state_valid = 0;
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_qk < 1 || D_qk > 256) return FLA_ERR_HEAD_DIM;
    if (D_v < 1 || D_v > 256) return FLA_ERR_V_HEAD_DIM;
    return chunked_forward({q, q_strides}, {k, k_strides}, {v, v_strides}, {o, o_strides}, B, H, N, D_qk, D_v, dtype,
                           state_out, state_valid, workspace, workspace_bytes, stream);
}

int fla_linear_attn_chunked_fwd_static(const void *q, const void *k, const void *v, void *o, int64_t B, int64_t H,
                                       int64_t N, int64_t D_qk, int64_t D_v, const int64_t *q_strides,
                                       const int64_t *k_strides, const int64_t *v_strides, const int64_t *o_strides,
                                       int dtype, void *stream) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_qk < 1 || D_qk > 256) return FLA_ERR_HEAD_DIM;
    if (D_v < 1 || D_v > 256) return FLA_ERR_V_HEAD_DIM;
    // what this call's kernels use of the workspace: without a state to hand over the walk path needs
    // the segments' entry states only; operands off that path take the 256-row chunks with their states
    const View vq{q, q_strides}, vk{k, k_strides}, vv{v, v_strides}, vo{o, o_strides};
    const View all[] = {vq, vk, vv, vo};
    for (const View &t : all)
        if (int rc = check_view(t)) return rc;
    const WalkPlan wp = walk_plan(B, H, N, D_qk, D_v, true);
    int64_t need = chunked_op_workspace_bytes(B, H, N, D_qk, D_v);
    if (wp.ok)
        need = fla::fast_path_ok(make_params(vq, vk, vv, vo, B, H, N, D_qk, D_v, 0)) ? wp.work_bytes
                                                                                      : chunked_bytes(B, H, N, D_qk, D_v);
    if (need > (int64_t)FLA_STATIC_SCRATCH_BYTES) return FLA_ERR_WORKSPACE;
    void *ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return chunked_forward({q, q_strides}, {k, k_strides}, {v, v_strides}, {o, o_strides}, B, H, N, D_qk, D_v, dtype,
                           nullptr, nullptr, ws, FLA_STATIC_SCRATCH_BYTES, stream);
}

int fla_feature_attn_fwd(const void *xq, const void *xk, const void *v, void *o, void *q_out, void *k_out, int64_t B,
                         int64_t H, int64_t N, int64_t D_qk, int64_t D_v, const int64_t *xq_strides,
                         const int64_t *xk_strides, const int64_t *v_strides, const int64_t *o_strides,
                         const int64_t *q_out_strides, const int64_t *k_out_strides, int feature_map, int dtype,
                         void *state_out, int32_t *state_valid, void *workspace, int64_t workspace_bytes, void *stream) {
    if (state_valid) *state_valid = 0;
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_qk < 1 || D_qk > 256) return FLA_ERR_HEAD_DIM;
    if (D_v < 1 || D_v > 256) return FLA_ERR_V_HEAD_DIM;
    if (feature_map != FLA_MAP_ELU1 && feature_map != FLA_MAP_SOFTPLUS) return FLA_ERR_UNSUPPORTED;
    const View mapped[2] = {{q_out, q_out_strides}, {k_out, k_out_strides}};
    return feature_forward({xq, xq_strides}, {xk, xk_strides}, {v, v_strides}, {o, o_strides}, mapped, B, H, N, D_qk, D_v,
                           feature_map, dtype, 1, state_out, state_valid, workspace, workspace_bytes, stream);
}

int fla_feature_attn_bwd(const void *grad_out, const void *xq, const void *xk, const void *v, void *dxq, void *dxk,
                         void *dv, int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                         const int64_t *go_strides, const int64_t *xq_strides, const int64_t *xk_strides,
                         const int64_t *v_strides, const int64_t *dxq_strides, const int64_t *dxk_strides,
                         const int64_t *dv_strides, int feature_map, int dtype, const void *state_in, void *workspace,
                         int64_t workspace_bytes, void *stream) {
    // (xq, xk name the forward's q_out, k_out here: phi(xq), phi(xk))
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_qk < 1 || D_qk > 256) return FLA_ERR_HEAD_DIM;
    if (D_v < 1 || D_v > 256) return FLA_ERR_V_HEAD_DIM;
    if (feature_map != FLA_MAP_ELU1 && feature_map != FLA_MAP_SOFTPLUS) return FLA_ERR_UNSUPPORTED;
    return chunked_backward({grad_out, go_strides}, {xq, xq_strides}, {xk, xk_strides}, {v, v_strides},
                            {dxq, dxq_strides}, {dxk, dxk_strides}, {dv, dv_strides}, B, H, N, D_qk, D_v, dtype,
                            state_in, workspace, workspace_bytes, stream, feature_map);
}

int fla_linear_attn_chunked_bwd(const void *grad_out, const void *q, const void *k, const void *v, void *dq, void *dk,
                                void *dv, int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                const int64_t *go_strides, const int64_t *q_strides, const int64_t *k_strides,
                                const int64_t *v_strides, const int64_t *dq_strides, const int64_t *dk_strides,
                                const int64_t *dv_strides, int dtype, const void *state_in, void *workspace,
                                int64_t workspace_bytes, void *stream) {
    if (int rc = check_common(B, H, N, dtype)) return rc;
    if (D_qk < 1 || D_qk > 256) return FLA_ERR_HEAD_DIM;
    if (D_v < 1 || D_v > 256) return FLA_ERR_V_HEAD_DIM;
    return chunked_backward({grad_out, go_strides}, {q, q_strides}, {k, k_strides}, {v, v_strides}, {dq, dq_strides},
                            {dk, dk_strides}, {dv, dv_strides}, B, H, N, D_qk, D_v, dtype, state_in, workspace,
                            workspace_bytes, stream);
}

int fla_feature_attn_normalised_fwd(const void *xq, const void *xk, const void *v, void *o, void *q_out, void *k_out,
                                    float *denom, int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                    const int64_t *xq_strides, const int64_t *xk_strides, const int64_t *v_strides,
                                    const int64_t *o_strides, const int64_t *q_out_strides,
                                    const int64_t *k_out_strides, int feature_map, float eps, int dtype, int chunked,
                                    void *state_out, int32_t *state_valid, void *workspace, int64_t workspace_bytes,
                                    void *stream) {
    if (state_valid) *state_valid = 0;
    if (int rc = check_norm_args(B, H, N, D_qk, D_v, dtype)) return rc;
    if (feature_map != FLA_MAP_ELU1 && feature_map != FLA_MAP_SOFTPLUS) return FLA_ERR_UNSUPPORTED;
    const View mapped[2] = {{q_out, q_out_strides}, {k_out, k_out_strides}};
    return normalised_forward({xq, xq_strides}, {xk, xk_strides}, {v, v_strides}, {o, o_strides}, denom, B, H, N, D_qk,
                              D_v, eps, dtype, chunked, workspace, workspace_bytes, stream, feature_map, mapped,
                              state_out, state_valid);
}

int fla_feature_attn_normalised_bwd(const void *grad_out, const void *q, const void *k, const void *v, const void *o,
                                    const float *denom, void *dxq, void *dxk, void *dv, int64_t B, int64_t H,
                                    int64_t N, int64_t D_qk, int64_t D_v, const int64_t *go_strides,
                                    const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                                    const int64_t *o_strides, const int64_t *dxq_strides, const int64_t *dxk_strides,
                                    const int64_t *dv_strides, int feature_map, int dtype, int chunked,
                                    const void *state_in, void *workspace, int64_t workspace_bytes, void *stream) {
    if (int rc = check_norm_args(B, H, N, D_qk, D_v, dtype)) return rc;
    if (feature_map != FLA_MAP_ELU1 && feature_map != FLA_MAP_SOFTPLUS) return FLA_ERR_UNSUPPORTED;
    return normalised_backward({grad_out, go_strides}, {q, q_strides}, {k, k_strides}, {v, v_strides}, {o, o_strides},
                               denom, {dxq, dxq_strides}, {dxk, dxk_strides}, {dv, dv_strides}, B, H, N, D_qk, D_v,
                               dtype, chunked, workspace, workspace_bytes, stream, feature_map, state_in);
}

int64_t fla_poly_attn_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t R, int64_t D_v) {
    if (B < 0 || H < 0 || N < 0 || R < 1 || R > 32 || D_v < 1 || D_v > 128) return 0;
    const PolyLayout l = poly_layout(B, H, N, R, D_v, 1);  // the normalised backward needs the most
    return 2 * l.packed_bytes + l.do_bytes + l.dn_bytes;
}

int fla_poly_attn_fwd(const void *xq, const void *xk, const void *v, void *o, float *denom, int64_t B, int64_t H,
                      int64_t N, int64_t R, int64_t D_v, const int64_t *xq_strides, const int64_t *xk_strides,
                      const int64_t *v_strides, const int64_t *o_strides, const float *coef, float eps, int dtype,
                      void *stream) {
    if (int rc = check_poly_args(B, H, N, R, D_v, dtype, coef)) return rc;
    return poly_forward({xq, xq_strides}, {xk, xk_strides}, {v, v_strides}, {o, o_strides}, denom, B, H, N, R, D_v,
                        coef, eps, dtype, stream);
}

int fla_poly_attn_bwd(const void *grad_out, const void *xq, const void *xk, const void *v, const void *o,
                      const float *denom, void *dxq, void *dxk, void *dv, int64_t B, int64_t H, int64_t N, int64_t R,
                      int64_t D_v, const int64_t *go_strides, const int64_t *xq_strides, const int64_t *xk_strides,
                      const int64_t *v_strides, const int64_t *o_strides, const int64_t *dxq_strides,
                      const int64_t *dxk_strides, const int64_t *dv_strides, const float *coef, int dtype,
                      void *workspace, int64_t workspace_bytes, void *stream) {
    if (int rc = check_poly_args(B, H, N, R, D_v, dtype, coef)) return rc;
    const View ov{o, o_strides};
    return poly_backward({grad_out, go_strides}, {xq, xq_strides}, {xk, xk_strides}, {v, v_strides},
                         o ? &ov : nullptr, denom, {dxq, dxq_strides}, {dxk, dxk_strides}, {dv, dv_strides}, B, H, N,
                         R, D_v, coef, dtype, workspace, workspace_bytes, stream);
}

int64_t fla_normalised_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v, int chunked) {
    if (B < 0 || H < 0 || N < 0 || D_qk < 1 || D_qk > 256 || D_v < 1 || D_v > 256) return 0;
    const NormLayout l = norm_layout(B, H, N, D_qk, D_v, chunked);
    return l.norm_bytes + l.chunk_bytes;
}

int fla_linear_attn_normalised_fwd(const void *q, const void *k, const void *v, void *o, float *denom, int64_t B,
                                   int64_t H, int64_t N, int64_t D_qk, int64_t D_v, const int64_t *q_strides,
                                   const int64_t *k_strides, const int64_t *v_strides, const int64_t *o_strides,
                                   float eps, int dtype, int chunked, void *state_out, int32_t *state_valid,
                                   void *workspace, int64_t workspace_bytes, void *stream) {
    if (state_valid) *state_valid = 0;
    if (int rc = check_norm_args(B, H, N, D_qk, D_v, dtype)) return rc;
    return normalised_forward({q, q_strides}, {k, k_strides}, {v, v_strides}, {o, o_strides}, denom, B, H, N, D_qk,
                              D_v, eps, dtype, chunked, workspace, workspace_bytes, stream, 0, nullptr, state_out,
                              state_valid);
}

int fla_linear_attn_normalised_bwd(const void *grad_out, const void *q, const void *k, const void *v, const void *o,
                                   const float *denom, void *dq, void *dk, void *dv, int64_t B, int64_t H,
                                   int64_t N, int64_t D_qk, int64_t D_v, const int64_t *go_strides,
                                   const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                                   const int64_t *o_strides, const int64_t *dq_strides, const int64_t *dk_strides,
                                   const int64_t *dv_strides, int dtype, int chunked, const void *state_in,
                                   void *workspace, int64_t workspace_bytes, void *stream) {
    if (int rc = check_norm_args(B, H, N, D_qk, D_v, dtype)) return rc;
    return normalised_backward({grad_out, go_strides}, {q, q_strides}, {k, k_strides}, {v, v_strides},
                               {o, o_strides}, denom, {dq, dq_strides}, {dk, dk_strides}, {dv, dv_strides}, B, H, N,
                               D_qk, D_v, dtype, chunked, workspace, workspace_bytes, stream, 0, state_in);
}

}  // extern "C"

#include "fla_trace_structs.h"  // (the trace build's descriptions of the parameter structs; empty otherwise)

/* fla.h -- C ABI of libfla_gfx950.so: causal linear attention O = tril(Q K^T) V,
 * forward and backward, as hand-written HIP kernels for gfx950 (MI355X).
 *
 * The reference has no native surface for this path: its four Python launch
 * wrappers JIT-compile Triton kernels.  Each entry point below replaces one of
 * those wrappers (cited per function); a Python binding passes
 * `tensor.data_ptr()`, `tensor.stride()` and the current stream's handle.
 *
 * Conventions
 *   - Every pointer is a device pointer on the current HIP device.
 *   - Tensors are 4-D, logical shape (B, H, N, D); `strides` is an array of 4
 *     element strides (b, h, n, d) and strides[3] must be 1.
 *   - `dtype` selects 16-bit storage: FLA_DTYPE_BF16 or FLA_DTYPE_F16.  Products
 *     run on bf16 / fp16 MFMA with fp32 accumulation; outputs are rounded once.
 *     Range of FLA_DTYPE_F16: the un-normalised product grows with N (an output element is a sum
 *     of up to N scores times values) and fp16 ends at 65504.  An output or gradient element
 *     whose fp32 value lies beyond that leaves as +inf or -inf, exactly as a cast of the fp32
 *     value would; finite inputs never produce NaN.  The masked scores are rounded to fp16 before
 *     the second product, so a single score q_i . k_j above 65504 becomes inf there (and inf * 0
 *     is NaN): keep |q_i . k_j| below that, e.g. by the usual 1/sqrt(D) scaling.  The chunk-wise
 *     entry points also round the running state (sums of k_j v_j^T over the rows before a chunk)
 *     to the storage type, so there the state's elements must fit as well.  The normalised
 *     entry points divide in fp32 before the one rounding: their outputs are averages of v and
 *     do not grow with N.  FLA_DTYPE_BF16 has fp32's exponent range and no such limit (the
 *     reference computes in bf16 only, flashlinear/kernels/linear_attn_kernels.py:82,98).
 *   - `stream` is a hipStream_t (NULL = the null stream).  Calls only enqueue
 *     work; they never synchronise, allocate or free.  Outputs must not alias
 *     inputs or each other: the byte range each tensor spans (first to last
 *     addressed element) is compared on the host and an overlap is rejected with
 *     FLA_ERR_ALIAS (the reference's wrappers always allocate fresh outputs,
 *     linear_attn_kernels.py:327, 366-368).
 *   - Re-entrant, no global mutable state (except the no-allocation variant
 *     documented at its declaration, if present).
 *   - Return value: FLA_OK or a negative FLA_ERR_* code; fla_strerror() names it.
 *     Nothing is enqueued when an error is returned.
 *   - N may be any non-negative value (the kernels bound-check rows).  The
 *     reference's "N % 64 == 0" precondition is enforced by the Python layer
 *     that mirrors the reference's asserts, not here.
 */
#ifndef FLA_H
#define FLA_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLA_ABI_VERSION 4

enum fla_dtype { FLA_DTYPE_BF16 = 0, FLA_DTYPE_F16 = 1 };

enum fla_status {
    FLA_OK = 0,
    FLA_ERR_NULL_POINTER = -1, /* a required pointer is NULL */
    FLA_ERR_DTYPE = -2,        /* dtype is not one of enum fla_dtype */
    FLA_ERR_HEAD_DIM = -3,     /* head dim < 1 or > 256 (linear_attn_kernels.py:322) */
    FLA_ERR_V_HEAD_DIM = -4,   /* small-V: D_v not a power of two, or next_pow2(D_v) > next_pow2(D_qk)
                                  (linear_attn_kernels_smallv_hd.py:336-337) */
    FLA_ERR_SHAPE = -5,        /* negative B, H or N, or B*H*N too large */
    FLA_ERR_STRIDE = -6,       /* strides[3] != 1, a NULL strides array, or a negative stride */
    FLA_ERR_LAUNCH = -7,       /* the HIP runtime rejected the launch */
    FLA_ERR_UNSUPPORTED = -8,  /* no kernel was built for this combination */
    FLA_ERR_WORKSPACE = -9,    /* chunked call: workspace missing, misaligned or too small */
    FLA_ERR_ALIAS = -10        /* an output tensor's byte range overlaps an input's or another output's */
};

/* ABI revision of the loaded library (== FLA_ABI_VERSION it was built with). */
int fla_abi_version(void);

/* Static, human-readable text for a status code. */
const char *fla_strerror(int status);

/* O = tril(Q K^T) V with equal head dims.
 * Replaces linear_flash_wrapper_fwd (flashlinear/kernels/linear_attn_kernels.py:310-341)
 * and the kernel it launches (linear_attn_kernels.py:11-100). */
int fla_linear_attn_fwd(const void *q, const void *k, const void *v, void *o,
                        int64_t B, int64_t H, int64_t N, int64_t D,
                        const int64_t *q_strides, const int64_t *k_strides,
                        const int64_t *v_strides, const int64_t *o_strides,
                        int dtype, void *stream);

/* dQ = tril(dO V^T) K,  dK = tril(dO V^T)^T Q,  dV = tril(Q K^T)^T dO, equal head dims.
 * Replaces linear_flash_wrapper_bwd (linear_attn_kernels.py:345-384) and
 * flash_attn_bwd (linear_attn_kernels.py:102-307).  Every element of dq, dk, dv
 * is written; no pre-zeroing is needed. */
int fla_linear_attn_bwd(const void *grad_out, const void *q, const void *k, const void *v,
                        void *dq, void *dk, void *dv,
                        int64_t B, int64_t H, int64_t N, int64_t D,
                        const int64_t *go_strides, const int64_t *q_strides,
                        const int64_t *k_strides, const int64_t *v_strides,
                        const int64_t *dq_strides, const int64_t *dk_strides,
                        const int64_t *dv_strides,
                        int dtype, void *stream);

/* Forward with q, k of width D_qk and v, o of width D_v (D_v a power of two,
 * next_pow2(D_v) <= next_pow2(D_qk)).
 * Replaces linear_flash_wrapper_fwd_smallv_hd
 * (flashlinear/kernels/linear_attn_kernels_smallv_hd.py:320-359) and its
 * kernel (linear_attn_kernels_smallv_hd.py:12-108). */
int fla_linear_attn_smallv_fwd(const void *q, const void *k, const void *v, void *o,
                               int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                               const int64_t *q_strides, const int64_t *k_strides,
                               const int64_t *v_strides, const int64_t *o_strides,
                               int dtype, void *stream);

/* Backward of the above.  Replaces linear_flash_wrapper_bwd_smallv_hd
 * (linear_attn_kernels_smallv_hd.py:363-405) and its kernel
 * (linear_attn_kernels_smallv_hd.py:111-317).  Like the reference's backward
 * wrapper it checks only D_qk <= 256 (linear_attn_kernels_smallv_hd.py:381). */
int fla_linear_attn_smallv_bwd(const void *grad_out, const void *q, const void *k, const void *v,
                               void *dq, void *dk, void *dv,
                               int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                               const int64_t *go_strides, const int64_t *q_strides,
                               const int64_t *k_strides, const int64_t *v_strides,
                               const int64_t *dq_strides, const int64_t *dk_strides,
                               const int64_t *dv_strides,
                               int dtype, void *stream);

/* The gradients of fla_linear_attn_bwd / fla_linear_attn_smallv_bwd evaluated the way the reference's
 * backward kernel does it in its first phase (linear_attn_kernels.py:160-227): a workgroup owns rows
 * of K and V and forms dV and dK from ONE stream of (Q, dO) tiles; dQ is a product of its own.
 * Equal padded head dims (32 / 64 / 128) with 16-byte aligned rows only, else FLA_ERR_UNSUPPORTED.
 * Results agree with fla_linear_attn_bwd (bit for bit up to padded width 64; up to the order of
 * fp32 sums at 128).  On MI355X this evaluation measured 4 - 16 % SLOWER than the three products in one
 * launch that fla_linear_attn_bwd makes, at every shape tried (the fused kernel halves the tile traffic
 * of two products but needs the whole register file of a SIMD for one wave, and the products are not
 * bound by that traffic), so nothing calls it by default; it is kept, tested and timed
 * (bench.py --bwd-plan fused-dkdv) as the measured alternative. */
int fla_linear_attn_bwd_fused_dkdv(const void *grad_out, const void *q, const void *k, const void *v,
                                   void *dq, void *dk, void *dv,
                                   int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                   const int64_t *go_strides, const int64_t *q_strides,
                                   const int64_t *k_strides, const int64_t *v_strides,
                                   const int64_t *dq_strides, const int64_t *dk_strides,
                                   const int64_t *dv_strides,
                                   int dtype, void *stream);

/* The one primitive all four calls above are built from:
 *
 *     Out = mask(X Y^T) Z        X, Y : (B, H, N, D_c)    Z, Out : (B, H, N, D_o)
 *
 * mask = lower triangle incl. diagonal when upper == 0 (row >= col), upper
 * triangle incl. diagonal when upper != 0 (row <= col).
 *     O  = lower(Q  K^T)  V      dQ = lower(dO V^T)  K
 *     dV = upper(K  Q^T)  dO     dK = upper(V  dO^T) Q
 * No counterpart in the reference (its kernels inline these four products,
 * linear_attn_kernels.py:74-82, 179-197, 291-299); exported for tests and
 * for callers that want a single gradient. */
int fla_tri_xyt_z(const void *x, const void *y, const void *z, void *out,
                  int64_t B, int64_t H, int64_t N, int64_t D_c, int64_t D_o,
                  const int64_t *x_strides, const int64_t *y_strides,
                  const int64_t *z_strides, const int64_t *out_strides,
                  int upper, int dtype, void *stream);

/* The same product evaluated chunk-wise: rows are cut into chunks of the kernel's row tile
 * (256 or 128 rows); each chunk's diagonal block is computed as above and everything off the
 * diagonal arrives through the running sum S of the per-chunk states Y_c^T Z_c (fp32,
 * rounded once to the storage dtype before X_c . S).  O(N (tile) D + N D_c D_o) work instead
 * of O(N^2 D): the algorithm of choice for long sequences.  Results differ from
 * fla_tri_xyt_z only by rounding.
 *
 * `workspace` is caller-owned device memory of at least fla_chunked_workspace_bytes() bytes,
 * 16-byte aligned; it is scratch (no need to clear it) and may be reused by the next call on
 * the same stream.  Operands that do not meet the fast-path alignment rules, and sequences
 * of a single chunk, are evaluated by fla_tri_xyt_z instead (workspace unused).
 * No counterpart in the reference: its kernels are quadratic in N
 * (linear_attn_kernels.py:63, 166-171). */
int64_t fla_chunked_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t D_c, int64_t D_o);
int fla_tri_xyt_z_chunked(const void *x, const void *y, const void *z, void *out,
                          int64_t B, int64_t H, int64_t N, int64_t D_c, int64_t D_o,
                          const int64_t *x_strides, const int64_t *y_strides,
                          const int64_t *z_strides, const int64_t *out_strides,
                          int upper, int dtype, void *workspace, int64_t workspace_bytes, void *stream);

/* The whole operator evaluated chunk-wise, forward and backward, with the running states
 * shared between products: O and dQ use the same state (sum of K_c^T V_c over earlier chunks),
 * dV and dK the same one (sum of Q_c^T dO_c over later chunks), so a forward + backward pair
 * computes two states instead of four.  Sharing needs operands that meet the speed-path alignment
 * rules and more than one chunk (more than 256 rows at padded head dims above 64); head dims are
 * padded to the next of 32 / 64 / 128, a D_qk up to 256 is taken as two 128-column halves and a D_v
 * up to 256 as two column halves of v.  Every other case evaluates each product with
 * fla_tri_xyt_z_chunked's method, same results.
 *
 * forward:  `state_out` (optional, fla_linear_attn_chunked_state_bytes() bytes, 16-byte aligned)
 *           receives what a later backward call can reuse of the running state (the fp32 state at
 *           the entry of every segment of the walk -- with two segments per (b, h), two partial
 *           sums whose sum is the second segment's -- and after the last chunk; the normalised
 *           operator at padded head dims up to 64: the rounded state at the entry of every
 *           chunk); *state_valid (host
 *           memory, optional) is set to 1 when it was written, else 0.
 * backward: `state_in` is that buffer, written by the forward call on the same q, k, v, or NULL
 *           (the state is then recomputed by another evaluation: two walks instead of one at
 *           padded head dims above 64, chunk states in memory below).
 * `workspace`: fla_linear_attn_chunked_workspace_bytes() bytes of scratch, 16-byte aligned.
 * No counterpart in the reference (quadratic kernels only, linear_attn_kernels.py:63, 166-171). */
int64_t fla_linear_attn_chunked_state_bytes(int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v);
/* 1 when fla_linear_attn_chunked_fwd + bwd are the faster pair for this shape on MI355X, 0 when the
 * quadratic fla_linear_attn(_smallv)_fwd + bwd are: a table of measured thresholds (host arithmetic,
 * no device call) in place of the autotuning the reference lists as a to-do (README.md:68). */
int fla_linear_attn_prefers_chunked(int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v);
int64_t fla_linear_attn_chunked_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v);
int fla_linear_attn_chunked_fwd(const void *q, const void *k, const void *v, void *o,
                                int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                const int64_t *q_strides, const int64_t *k_strides,
                                const int64_t *v_strides, const int64_t *o_strides,
                                int dtype, void *state_out, int32_t *state_valid,
                                void *workspace, int64_t workspace_bytes, void *stream);
int fla_linear_attn_chunked_bwd(const void *grad_out, const void *q, const void *k, const void *v,
                                void *dq, void *dk, void *dv,
                                int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                const int64_t *go_strides, const int64_t *q_strides,
                                const int64_t *k_strides, const int64_t *v_strides,
                                const int64_t *dq_strides, const int64_t *dk_strides,
                                const int64_t *dv_strides,
                                int dtype, const void *state_in,
                                void *workspace, int64_t workspace_bytes, void *stream);

/* Causal linear attention on q = phi(xq), k = phi(xk) for an element-wise feature map phi,
 *
 *     O = tril(phi(Xq) phi(Xk)^T) V,
 *
 * evaluated chunk-wise (fla_linear_attn_chunked_fwd/bwd's method) with phi applied while the
 * kernels load xq and xk: the kernel that builds the chunk states maps xk as its tiles arrive,
 * the main kernel maps its rows of xq, and each writes what it mapped to q_out = phi(xq),
 * k_out = phi(xk) ((B, H, N, D_qk) in the storage dtype; every element is written) -- a
 * by-product that replaces xq, xk as what backward needs, so no pass over memory exists for the
 * map alone.  Backward takes q = q_out, k = k_out and returns the gradients with respect to xq
 * and xk directly,
 *     dXq = (tril(dO V^T) K) . phi'(Xq),    dXk = (tril(dO V^T)^T Q) . phi'(Xk),    dV,
 * the slopes computed from q, k themselves (elu(x) + 1: 1 where y >= 1, else y; softplus:
 * 1 - e^-y) and multiplied into the accumulators before they are rounded and stored.
 * feature_map: FLA_MAP_ELU1 (elu(x) + 1) or FLA_MAP_SOFTPLUS (log(1 + e^x), the map the
 * reference's tests put in front of its operators, flashlinear/test_attn.py:36-40); phi is
 * evaluated in fp32 and rounded once to the storage dtype.  state_out / state_valid / state_in,
 * workspace: exactly as for fla_linear_attn_chunked_fwd/bwd, same size queries.  Shapes and
 * layouts outside the shared-state fast path (unequal padded head dims, a single chunk,
 * unaligned operands) run an element-wise pass per operand instead, same results.  No
 * counterpart in the reference: its callers materialise phi(x) with PyTorch passes before the
 * operator and differentiate through them with more (README.md:27-30 of the reference). */
enum fla_feature_map { FLA_MAP_NONE = 0, FLA_MAP_ELU1 = 1, FLA_MAP_SOFTPLUS = 2 };
int fla_feature_attn_fwd(const void *xq, const void *xk, const void *v, void *o, void *q_out, void *k_out,
                         int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                         const int64_t *xq_strides, const int64_t *xk_strides,
                         const int64_t *v_strides, const int64_t *o_strides,
                         const int64_t *q_out_strides, const int64_t *k_out_strides,
                         int feature_map, int dtype, void *state_out, int32_t *state_valid,
                         void *workspace, int64_t workspace_bytes, void *stream);
int fla_feature_attn_bwd(const void *grad_out, const void *q, const void *k, const void *v,
                         void *dxq, void *dxk, void *dv,
                         int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                         const int64_t *go_strides, const int64_t *q_strides,
                         const int64_t *k_strides, const int64_t *v_strides,
                         const int64_t *dxq_strides, const int64_t *dxk_strides,
                         const int64_t *dv_strides,
                         int feature_map, int dtype, const void *state_in,
                         void *workspace, int64_t workspace_bytes, void *stream);

/* The two operators above combined: normalised causal linear attention on q = phi(xq),
 * k = phi(xk),   out_i = [tril(Q K^T) V]_i / (q_i . (k_0 + ... + k_i) + eps),
 * arguments as for fla_linear_attn_normalised_fwd/bwd (same workspace size query, `chunked`
 * selects the product's evaluation) plus the feature map and its by-products q_out, k_out as for
 * fla_feature_attn_fwd.  With the chunk-wise product the map is applied while the kernels load
 * xq, xk; with the quadratic kernels by one element-wise pass per operand.  Backward takes
 * q = q_out, k = k_out and returns gradients with respect to xq, xk: the slope of phi is
 * multiplied in by the pass that adds the normaliser's own terms.  No counterpart in the
 * reference (README.md:27-30 of the reference is the recipe this replaces). */
int fla_feature_attn_normalised_fwd(const void *xq, const void *xk, const void *v, void *o, void *q_out, void *k_out,
                                    float *denom,
                                    int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                    const int64_t *xq_strides, const int64_t *xk_strides,
                                    const int64_t *v_strides, const int64_t *o_strides,
                                    const int64_t *q_out_strides, const int64_t *k_out_strides,
                                    int feature_map, float eps, int dtype, int chunked,
                                    void *state_out, int32_t *state_valid,
                                    void *workspace, int64_t workspace_bytes, void *stream);
int fla_feature_attn_normalised_bwd(const void *grad_out, const void *q, const void *k, const void *v,
                                    const void *o, const float *denom, void *dxq, void *dxk, void *dv,
                                    int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                    const int64_t *go_strides, const int64_t *q_strides,
                                    const int64_t *k_strides, const int64_t *v_strides,
                                    const int64_t *o_strides, const int64_t *dxq_strides,
                                    const int64_t *dxk_strides, const int64_t *dv_strides,
                                    int feature_map, int dtype, int chunked, const void *state_in,
                                    void *workspace, int64_t workspace_bytes, void *stream);

/* fla_linear_attn_chunked_fwd for callers that cannot allocate device memory or pass a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments and results as fla_linear_attn_chunked_fwd with
 * state_out = NULL; the scratch its kernels need (per-chunk states and their running sums) lives
 * in a static device array of FLA_STATIC_SCRATCH_BYTES that every GPU the library runs on holds
 * until the process ends.  The call allocates and frees nothing.  A problem whose kernels need more
 * scratch than FLA_STATIC_SCRATCH_BYTES is rejected with FLA_ERR_WORKSPACE before anything is
 * enqueued.  What they need depends on the path the operands take: equal padded head dims up to 128
 * with 16-byte aligned rows use the segments' fp32 entry states only (at most 256 (D <= 64: 512)
 * states of D x D, 16 MiB at D = 128, whatever B, H and N); other shapes and layouts use the
 * per-chunk states, fla_chunked_workspace_bytes() or, for D_qk in (128, 256] with D_v <= 128,
 * fla_linear_attn_chunked_workspace_bytes().  All calls on one GPU share that array (it keeps
 * the previous call's contents; the kernels overwrite what they read): calls that overlap in
 * time on one GPU -- different streams, different host threads -- race; calls on one stream do not. */
#define FLA_STATIC_SCRATCH_BYTES (64 * 1024 * 1024)
int fla_linear_attn_chunked_fwd_static(const void *q, const void *k, const void *v, void *o,
                                       int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                       const int64_t *q_strides, const int64_t *k_strides,
                                       const int64_t *v_strides, const int64_t *o_strides,
                                       int dtype, void *stream);

/* Causal linear attention with a polynomial score map,
 *
 *     out = lower(f(Xq Xk^T)) V,    f(u) = coef[0] + coef[1] u + coef[2] u^2,
 *
 * i.e. LinearAttentionSmallVHD on second-order Taylor features phi(x) with
 * phi(x) . phi(y) = f(x . y) (the reference's README.md:3 use case: 256 features from a 16-wide
 * x, coef = {0, 0, 1/2}; the full Taylor map is {1, 1, 1/2}) -- with the features never built:
 * scores cost an R-wide contraction instead of an R^2-wide one.  xq, xk: (B, H, N, R), R <= 32;
 * v, o: (B, H, N, D_v), D_v <= 128.  When `denom` is non-NULL the output rows are divided by
 * n = (row sum of the masked scores) + eps and n is stored there (fp32, contiguous (B, H, N)).
 * Backward forms
 *     dV  = upper(f(Xk Xq^T)) dO
 *     dXq = lower((dO V^T) . f'(Xq Xk^T)) Xk,   dXk = upper((V dO^T) . f'(Xk Xq^T)) Xq
 * and needs fla_poly_attn_workspace_bytes() bytes of 16-byte aligned scratch.  For the
 * normalised forward pass the forward's `o` and `denom` to backward (both NULL otherwise): dO
 * becomes g / n, and the normaliser's own gradient dn = -(g . o) / n enters the first score of
 * dXq and dXk as a bias (dO V^T + dn 1^T); B*H must then not exceed 65535.  Fast-path kernels
 * only: every operand 16-byte aligned with widths and outer strides multiples of 8 elements,
 * else FLA_ERR_UNSUPPORTED.  No counterpart in the reference (it multiplies materialised
 * features, linear_attn_kernels_smallv_hd.py:78-86). */
int64_t fla_poly_attn_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t R, int64_t D_v);
int fla_poly_attn_fwd(const void *xq, const void *xk, const void *v, void *o, float *denom,
                      int64_t B, int64_t H, int64_t N, int64_t R, int64_t D_v,
                      const int64_t *xq_strides, const int64_t *xk_strides,
                      const int64_t *v_strides, const int64_t *o_strides,
                      const float *coef, float eps, int dtype, void *stream);
int fla_poly_attn_bwd(const void *grad_out, const void *xq, const void *xk, const void *v,
                      const void *o, const float *denom,
                      void *dxq, void *dxk, void *dv,
                      int64_t B, int64_t H, int64_t N, int64_t R, int64_t D_v,
                      const int64_t *go_strides, const int64_t *xq_strides,
                      const int64_t *xk_strides, const int64_t *v_strides, const int64_t *o_strides,
                      const int64_t *dxq_strides, const int64_t *dxk_strides,
                      const int64_t *dv_strides,
                      const float *coef, int dtype, void *workspace, int64_t workspace_bytes, void *stream);

/* Normalised causal linear attention, the full operator a caller of the reference assembles
 * in PyTorch around LinearAttention.apply (README.md:27-30 of the reference):
 *
 *     n_i = q_i . (k_0 + ... + k_i) + eps        out_i = [tril(Q K^T) V]_i / n_i
 *
 * Forward runs the product above and then one fused pass that forms n (cumulative sum of k,
 * dot with q, eps) and divides in place; `denom` receives n as fp32, contiguous (B, H, N), for
 * the backward call.  Backward takes d(out), the forward's `o` and `denom`, and returns the
 * gradients of q, k, v including the normaliser's own terms.  D_qk and D_v are independent
 * (1..256).  `chunked` != 0 evaluates the products chunk-wise (fla_linear_attn_chunked_fwd/bwd's
 * method) instead of with the quadratic kernels.  `workspace`: at least
 * fla_normalised_workspace_bytes() bytes (same `chunked`) of 16-byte aligned device memory,
 * scratch.  state_out / state_valid / state_in: with `chunked`, what the chunk-wise forward hands to
 * its backward, exactly as for fla_linear_attn_chunked_fwd/bwd (size:
 * fla_linear_attn_chunked_state_bytes(); any of them may be null, backward then works without;
 * state_in must be what THIS operator's forward wrote for the same inputs -- behind the product's
 * state it carries the running sums of k, which the plain chunk-wise forward does not write);
 * ignored otherwise.  With `chunked` and equal padded head dims up to 128 the normaliser and
 * its gradient terms are computed inside the chunk-wise kernels rather than by passes of their
 * own.  B*H must not exceed 65535.  No counterpart in the reference's kernels; replaces the caller-side recipe and its
 * autograd graph (a cumsum, two elementwise products, a row sum and a division, each a full
 * pass over memory, forward and backward). */
int64_t fla_normalised_workspace_bytes(int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v, int chunked);
int fla_linear_attn_normalised_fwd(const void *q, const void *k, const void *v, void *o, float *denom,
                                   int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                   const int64_t *q_strides, const int64_t *k_strides,
                                   const int64_t *v_strides, const int64_t *o_strides,
                                   float eps, int dtype, int chunked,
                                   void *state_out, int32_t *state_valid,
                                   void *workspace, int64_t workspace_bytes, void *stream);
int fla_linear_attn_normalised_bwd(const void *grad_out, const void *q, const void *k, const void *v,
                                   const void *o, const float *denom, void *dq, void *dk, void *dv,
                                   int64_t B, int64_t H, int64_t N, int64_t D_qk, int64_t D_v,
                                   const int64_t *go_strides, const int64_t *q_strides,
                                   const int64_t *k_strides, const int64_t *v_strides,
                                   const int64_t *o_strides, const int64_t *dq_strides,
                                   const int64_t *dk_strides, const int64_t *dv_strides,
                                   int dtype, int chunked, const void *state_in,
                                   void *workspace, int64_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* FLA_H */

/* Brute-force C restatement of un-normalised causal linear attention.
 *
 * TEST INFRASTRUCTURE ONLY: linked by tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py as the checker; never by the product library.
 *
 * Triple loops straight from the definitions, double accumulation, no tiling:
 *
 *   o[i,e]  = sum_{j<=i} (sum_d q[i,d] k[j,d]) v[j,e]
 *             (flashlinear/kernels/linear_attn_kernels.py:63-82: loop over key
 *              tiles up to the diagonal, mask row >= col, accumulate S V)
 *   dv[j,e] = sum_{i>=j} (q_i . k_j) do[i,e]
 *             (linear_attn_kernels.py:179-187)
 *   dk[j,d] = sum_{i>=j} (do_i . v_j) q[i,d]
 *             (linear_attn_kernels.py:189-197)
 *   dq[i,d] = sum_{j<=i} (do_i . v_j) k[j,d]
 *             (linear_attn_kernels.py:291-299)
 *
 * Layout: contiguous (BH, N, D) float32 arrays; every bh slice independent
 * (linear_attn_kernels.py:21-27).  d_qk and d_v may differ
 * (flashlinear/kernels/linear_attn_kernels_smallv_hd.py:326-327).
 */
#include <stddef.h>
#include <stdlib.h>

static double dot(const float *a, const float *b, int d)
{
    double s = 0.0;
    for (int x = 0; x < d; ++x)
        s += (double)a[x] * (double)b[x];
    return s;
}

int oracle_causal_dot_product_fwd(const float *q, const float *k, const float *v, float *o,
                                  long bh, int n, int d_qk, int d_v)
{
    if (!q || !k || !v || !o || bh < 0 || n < 0 || d_qk <= 0 || d_v <= 0)
        return -1;
    double *acc = (double *)malloc(sizeof(double) * (size_t)d_v);
    if (!acc)
        return -2;
    for (long s = 0; s < bh; ++s) {
        const float *qs = q + (size_t)s * n * d_qk, *ks = k + (size_t)s * n * d_qk;
        const float *vs = v + (size_t)s * n * d_v;
        float *os = o + (size_t)s * n * d_v;
        for (int i = 0; i < n; ++i) {
            for (int e = 0; e < d_v; ++e)
                acc[e] = 0.0;
            for (int j = 0; j <= i; ++j) {
                double a = dot(qs + (size_t)i * d_qk, ks + (size_t)j * d_qk, d_qk);
                for (int e = 0; e < d_v; ++e)
                    acc[e] += a * (double)vs[(size_t)j * d_v + e];
            }
            for (int e = 0; e < d_v; ++e)
                os[(size_t)i * d_v + e] = (float)acc[e];
        }
    }
    free(acc);
    return 0;
}

int oracle_causal_dot_product_bwd(const float *q, const float *k, const float *v, const float *go,
                                  float *dq, float *dk, float *dv,
                                  long bh, int n, int d_qk, int d_v)
{
    if (!q || !k || !v || !go || !dq || !dk || !dv || bh < 0 || n < 0 || d_qk <= 0 || d_v <= 0)
        return -1;
    int dmax = d_qk > d_v ? d_qk : d_v;
    double *acc = (double *)malloc(sizeof(double) * (size_t)dmax * 2);
    if (!acc)
        return -2;
    double *acc2 = acc + dmax;
    for (long s = 0; s < bh; ++s) {
        const float *qs = q + (size_t)s * n * d_qk, *ks = k + (size_t)s * n * d_qk;
        const float *vs = v + (size_t)s * n * d_v, *gs = go + (size_t)s * n * d_v;
        float *dqs = dq + (size_t)s * n * d_qk, *dks = dk + (size_t)s * n * d_qk;
        float *dvs = dv + (size_t)s * n * d_v;
        /* key-side gradients: row j gathers from queries i >= j */
        for (int j = 0; j < n; ++j) {
            for (int x = 0; x < d_v; ++x)
                acc[x] = 0.0;
            for (int x = 0; x < d_qk; ++x)
                acc2[x] = 0.0;
            for (int i = j; i < n; ++i) {
                double a = dot(qs + (size_t)i * d_qk, ks + (size_t)j * d_qk, d_qk);
                double m = dot(gs + (size_t)i * d_v, vs + (size_t)j * d_v, d_v);
                for (int e = 0; e < d_v; ++e)
                    acc[e] += a * (double)gs[(size_t)i * d_v + e];
                for (int d = 0; d < d_qk; ++d)
                    acc2[d] += m * (double)qs[(size_t)i * d_qk + d];
            }
            for (int e = 0; e < d_v; ++e)
                dvs[(size_t)j * d_v + e] = (float)acc[e];
            for (int d = 0; d < d_qk; ++d)
                dks[(size_t)j * d_qk + d] = (float)acc2[d];
        }
        /* query-side gradient: row i gathers from keys j <= i */
        for (int i = 0; i < n; ++i) {
            for (int x = 0; x < d_qk; ++x)
                acc2[x] = 0.0;
            for (int j = 0; j <= i; ++j) {
                double m = dot(gs + (size_t)i * d_v, vs + (size_t)j * d_v, d_v);
                for (int d = 0; d < d_qk; ++d)
                    acc2[d] += m * (double)ks[(size_t)j * d_qk + d];
            }
            for (int d = 0; d < d_qk; ++d)
                dqs[(size_t)i * d_qk + d] = (float)acc2[d];
        }
    }
    free(acc);
    return 0;
}

/*
 * CPU oracle, C restatement: TEST INFRASTRUCTURE, not product code.  Only tests and the
 * smoke check may load the library built from this file; the product never does.
 *
 * Evoformer attention forward and backward in double precision with plain loops, one
 * score at a time.  It follows the formula the reference checks itself against
 * (dsevoformer-triton/test.py:47-57):
 *     s_ij = scale * <q_i, k_j> + bias[b,h,i,j] + mask[b,s,j]
 *     p_ij = exp(s_ij - lse_i),  lse_i = log sum_j exp(s_ij)      (evoformer.py:285-288)
 *     o_i  = sum_j p_ij v_j
 * and the textbook softmax-attention backward the reference's kernels implement
 * (evoformer.py:313-323 delta, :450-462 dS/dQ/dBias, :594-614 dV/dK):
 *     delta_i = <do_i, o_i>; dp_ij = <do_i, v_j>; ds_ij = p_ij (dp_ij - delta_i)
 *     dq_i = scale sum_j ds_ij k_j; dk_j = scale sum_i ds_ij q_i; dv_j = sum_i p_ij do_i
 *     dbias[b,h,i,j] = sum_s ds_ij;  dmask[b,s,j] = sum_{h,i} ds_ij
 * Operands are head-major and dense: q,k,v,o,do,dq,dk,dv [B][H][S][N][D],
 * bias,dbias [B][H][N][N] (may be NULL), mask,dmask [B][S][N] additive (may be NULL),
 * lse [B][H][S][N].  A bool keep-mask is passed as 0 / -DBL_MAX-like additive values by
 * the caller.  The mapping from the [B,S,N,H,D] interface layout to head-major is done by
 * the caller so that this file stays an independent check of the arithmetic only.
 *
 * Pinned by tests/test_oracle.py against closed forms and a numpy brute force.
 */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>

static double dot(const double *a, const double *b, int n) {
    double s = 0.0;
    for (int i = 0; i < n; ++i) s += a[i] * b[i];
    return s;
}

/* scores of one query row against all keys, with bias and mask applied */
static void score_row(const double *q, const double *k, const double *bias_row,
                      const double *mask_row, int N, int D, double scale, double *s) {
    for (int j = 0; j < N; ++j) {
        double v = scale * dot(q, k + (size_t)j * D, D);
        if (bias_row) v += bias_row[j];
        if (mask_row) v += mask_row[j];
        s[j] = v;
    }
}

static double logsumexp(const double *s, int N) {
    double m = s[0];
    for (int j = 1; j < N; ++j) if (s[j] > m) m = s[j];
    double l = 0.0;
    for (int j = 0; j < N; ++j) l += exp(s[j] - m);
    return m + log(l);
}

int evo_ref_fwd(const double *q, const double *k, const double *v, const double *bias,
                const double *mask, int B, int H, int S, int N, int D, double scale,
                double *o, double *lse) {
    double *s = (double *)malloc(sizeof(double) * (size_t)N);
    if (!s) return -1;
    for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h)
    for (int si = 0; si < S; ++si) {
        size_t prob = ((size_t)b * H + h) * S + si;
        const double *qp = q + prob * N * D, *kp = k + prob * N * D, *vp = v + prob * N * D;
        const double *mrow = mask ? mask + ((size_t)b * S + si) * N : NULL;
        for (int i = 0; i < N; ++i) {
            const double *brow = bias ? bias + (((size_t)b * H + h) * N + i) * N : NULL;
            score_row(qp + (size_t)i * D, kp, brow, mrow, N, D, scale, s);
            double L = logsumexp(s, N);
            lse[prob * N + i] = L;
            double *op = o + (prob * N + i) * D;
            for (int d = 0; d < D; ++d) op[d] = 0.0;
            for (int j = 0; j < N; ++j) {
                double p = exp(s[j] - L);
                for (int d = 0; d < D; ++d) op[d] += p * vp[(size_t)j * D + d];
            }
        }
    }
    free(s);
    return 0;
}

int evo_ref_bwd(const double *q, const double *k, const double *v, const double *bias,
                const double *mask, const double *dout, int B, int H, int S, int N, int D,
                double scale, double *dq, double *dk, double *dv, double *dbias,
                double *dmask) {
    double *s = (double *)malloc(sizeof(double) * (size_t)N);
    double *orow = (double *)malloc(sizeof(double) * (size_t)D);
    if (!s || !orow) { free(s); free(orow); return -1; }
    size_t tot = (size_t)B * H * S * N * D;
    for (size_t t = 0; t < tot; ++t) { dq[t] = 0.0; dk[t] = 0.0; dv[t] = 0.0; }
    if (dbias) for (size_t t = 0; t < (size_t)B * H * N * N; ++t) dbias[t] = 0.0;
    if (dmask) for (size_t t = 0; t < (size_t)B * S * N; ++t) dmask[t] = 0.0;
    for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h)
    for (int si = 0; si < S; ++si) {
        size_t prob = ((size_t)b * H + h) * S + si;
        const double *qp = q + prob * N * D, *kp = k + prob * N * D, *vp = v + prob * N * D;
        const double *gp = dout + prob * N * D;
        const double *mrow = mask ? mask + ((size_t)b * S + si) * N : NULL;
        for (int i = 0; i < N; ++i) {
            const double *brow = bias ? bias + (((size_t)b * H + h) * N + i) * N : NULL;
            score_row(qp + (size_t)i * D, kp, brow, mrow, N, D, scale, s);
            double L = logsumexp(s, N);
            for (int d = 0; d < D; ++d) orow[d] = 0.0;
            for (int j = 0; j < N; ++j) {
                double p = exp(s[j] - L);
                for (int d = 0; d < D; ++d) orow[d] += p * vp[(size_t)j * D + d];
            }
            double delta = dot(gp + (size_t)i * D, orow, D);
            for (int j = 0; j < N; ++j) {
                double p = exp(s[j] - L);
                double dp = dot(gp + (size_t)i * D, vp + (size_t)j * D, D);
                double ds = p * (dp - delta);
                for (int d = 0; d < D; ++d) {
                    dv[(prob * N + j) * D + d] += p * gp[(size_t)i * D + d];
                    dq[(prob * N + i) * D + d] += scale * ds * kp[(size_t)j * D + d];
                    dk[(prob * N + j) * D + d] += scale * ds * qp[(size_t)i * D + d];
                }
                if (dbias) dbias[(((size_t)b * H + h) * N + i) * N + j] += ds;
                if (dmask) dmask[((size_t)b * S + si) * N + j] += ds;
            }
        }
    }
    free(s); free(orow);
    return 0;
}

/* CPU oracle for TaH duo-causal attention on the packed varlen layout.
 * TEST INFRASTRUCTURE ONLY: nothing shipped links or loads this file.
 *
 * Double-precision accumulation, float32 in/out, plain loops.  Written
 * independently of oracle/duo_oracle.py so the two can check each other:
 * forward = per-row two-pass softmax; backward = the analytic gradient of
 * softmax(QK^T s + M)V (no autograd).
 *
 * Visibility (tah/model/tah_model.py:788): key (kp, kd) is visible to query
 * (qp, qd) iff kp <= qp and kd <= qd.  Depth-0 key j of a sequence has
 * position j; depth-0 query i has position i + (Lk1 - Lq1); depth-1 rows carry
 * explicit positions.  GQA: q head h reads kv head h / (Hq/Hkv)
 * (transformers/integrations/sdpa_attention.py:15-24).  Depth-0 K/V receive
 * gradient from both query streams (tah/model/causal_cache.py:92-93 keeps the
 * cached tensors attached to the graph).
 *
 * Build: see oracle/Makefile  ->  oracle/libduo_ref.so
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    const float *q, *k1, *v1, *k2, *v2;
    int D;
} row_ctx;

/* scores of one query row against the visible prefix of both key segments */
static double row_scores(const float *q, const float *k1, long n1, const float *k2,
                         const int *pos2, long n2_all, long qpos, long kstride, int D,
                         double scale, double *s, long *n2_out)
{
    double m = -INFINITY;
    long n = 0;
    for (long j = 0; j < n1; ++j) {
        const float *kr = k1 + j * kstride;
        double acc = 0.0;
        for (int d = 0; d < D; ++d) acc += (double)q[d] * (double)kr[d];
        s[n] = acc * scale;
        if (s[n] > m) m = s[n];
        ++n;
    }
    long n2 = 0;
    for (long j = 0; j < n2_all; ++j) {
        if ((long)pos2[j] > qpos) { s[n1 + j] = -INFINITY; continue; }
        const float *kr = k2 + j * kstride;
        double acc = 0.0;
        for (int d = 0; d < D; ++d) acc += (double)q[d] * (double)kr[d];
        s[n1 + j] = acc * scale;
        if (s[n1 + j] > m) m = s[n1 + j];
        ++n2;
    }
    *n2_out = n2;
    return m;
}

static long clampl(long x, long lo, long hi) { return x < lo ? lo : (x > hi ? hi : x); }

/* One query stream (depth 0 when k2 == NULL / see2 == 0, depth 1 otherwise). */
static void stream_fwd(const float *q, long q0, long q1_, const int *qpos_arr, long qoff,
                       const float *k1, const float *v1, long c0, long lk1,
                       const float *k2, const float *v2, const int *pos_k2, long e0, long lk2,
                       int see2, int Hq, int Hkv, int D, int hk, double scale,
                       float *o, float *lse, long lse_stride, double *s, double *acc)
{
    int g = Hq / Hkv;
    long kstride = (long)Hkv * D;
    for (long i = q0; i < q1_; ++i) {
        long p = qpos_arr ? (long)qpos_arr[i] : (i - q0) + qoff;
        long n1 = clampl(p + 1, 0, lk1);
        for (int hh = 0; hh < g; ++hh) {
            int h = hk * g + hh;
            const float *qr = q + (i * Hq + h) * D;
            long n2;
            double m = row_scores(qr, k1 + (c0 * Hkv + hk) * D, n1,
                                  see2 ? k2 + (e0 * Hkv + hk) * D : NULL, pos_k2 ? pos_k2 + e0 : NULL,
                                  see2 ? lk2 : 0, p, kstride, D, scale, s, &n2);
            float *orow = o + (i * Hq + h) * D;
            if (n1 + n2 == 0) {
                memset(orow, 0, sizeof(float) * D);
                lse[h * lse_stride + i] = -INFINITY;
                continue;
            }
            for (int d = 0; d < D; ++d) acc[d] = 0.0;
            double l = 0.0;
            for (long j = 0; j < n1; ++j) {
                double e = exp(s[j] - m);
                l += e;
                const float *vr = v1 + ((c0 + j) * Hkv + hk) * D;
                for (int d = 0; d < D; ++d) acc[d] += e * (double)vr[d];
            }
            for (long j = 0; see2 && j < lk2; ++j) {
                if (s[n1 + j] == -INFINITY) continue;
                double e = exp(s[n1 + j] - m);
                l += e;
                const float *vr = v2 + ((e0 + j) * Hkv + hk) * D;
                for (int d = 0; d < D; ++d) acc[d] += e * (double)vr[d];
            }
            for (int d = 0; d < D; ++d) orow[d] = (float)(acc[d] / l);
            lse[h * lse_stride + i] = (float)(m + log(l));
        }
    }
}

int duo_ref_fwd(const float *q1, const float *k1, const float *v1, const int *cu_q1,
                const int *cu_k1, const float *q2, const float *k2, const float *v2,
                const int *pos_q2, const int *pos_k2, const int *cu_q2, const int *cu_k2,
                int nseq, int Hq, int Hkv, int D, float scale_f,
                float *o1, float *lse1, float *o2, float *lse2)
{
    if (Hq % Hkv) return -1;
    double scale = (double)scale_f;
    long T1q = cu_q1[nseq], T2q = cu_q2[nseq];
    long maxk = 0;
    for (int b = 0; b < nseq; ++b) {
        long n = (cu_k1[b + 1] - cu_k1[b]) + (cu_k2[b + 1] - cu_k2[b]);
        if (n > maxk) maxk = n;
    }
    int fail = 0;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int b = 0; b < nseq; ++b) {
        for (int hk = 0; hk < Hkv; ++hk) {
            double *s = (double *)malloc(sizeof(double) * (size_t)(maxk + 1));
            double *acc = (double *)malloc(sizeof(double) * (size_t)D);
            if (!s || !acc) { fail = 1; free(s); free(acc); continue; }
            long lq1 = cu_q1[b + 1] - cu_q1[b], lk1 = cu_k1[b + 1] - cu_k1[b];
            stream_fwd(q1, cu_q1[b], cu_q1[b + 1], NULL, lk1 - lq1, k1, v1, cu_k1[b], lk1,
                       NULL, NULL, NULL, 0, 0, 0, Hq, Hkv, D, hk, scale, o1, lse1, T1q, s, acc);
            stream_fwd(q2, cu_q2[b], cu_q2[b + 1], pos_q2, 0, k1, v1, cu_k1[b], lk1,
                       k2, v2, pos_k2, cu_k2[b], cu_k2[b + 1] - cu_k2[b], 1, Hq, Hkv, D, hk,
                       scale, o2, lse2, T2q, s, acc);
            free(s);
            free(acc);
        }
    }
    return fail ? -2 : 0;
}

/* Analytic backward of one query stream; dk/dv accumulators are double and
 * owned by the calling (b, hk) iteration, so no two threads share a row. */
static void stream_bwd(const float *q, const float *dout, long q0, long q1_, const int *qpos_arr,
                       long qoff, const float *k1, const float *v1, long c0, long lk1,
                       const float *k2, const float *v2, const int *pos_k2, long e0, long lk2,
                       int see2, int Hq, int Hkv, int D, int hk, double scale,
                       float *dq, double *dk1, double *dv1, double *dk2, double *dv2,
                       double *s, double *acc)
{
    int g = Hq / Hkv;
    long kstride = (long)Hkv * D;
    double *dqa = acc;          /* D */
    double *oa = acc + D;       /* D */
    for (long i = q0; i < q1_; ++i) {
        long p = qpos_arr ? (long)qpos_arr[i] : (i - q0) + qoff;
        long n1 = clampl(p + 1, 0, lk1);
        for (int hh = 0; hh < g; ++hh) {
            int h = hk * g + hh;
            const float *qr = q + (i * Hq + h) * D;
            const float *go = dout + (i * Hq + h) * D;
            float *dqr = dq + (i * Hq + h) * D;
            long n2;
            double m = row_scores(qr, k1 + (c0 * Hkv + hk) * D, n1,
                                  see2 ? k2 + (e0 * Hkv + hk) * D : NULL, pos_k2 ? pos_k2 + e0 : NULL,
                                  see2 ? lk2 : 0, p, kstride, D, scale, s, &n2);
            if (n1 + n2 == 0) { memset(dqr, 0, sizeof(float) * D); continue; }
            long ntot = n1 + (see2 ? lk2 : 0);
            double l = 0.0;
            for (long j = 0; j < ntot; ++j) {
                s[j] = (s[j] == -INFINITY) ? 0.0 : exp(s[j] - m);
                l += s[j];
            }
            for (int d = 0; d < D; ++d) { oa[d] = 0.0; dqa[d] = 0.0; }
            for (long j = 0; j < ntot; ++j) {
                s[j] /= l; /* probabilities */
                if (s[j] == 0.0) continue;
                const float *vr = (j < n1) ? v1 + ((c0 + j) * Hkv + hk) * D
                                           : v2 + ((e0 + (j - n1)) * Hkv + hk) * D;
                for (int d = 0; d < D; ++d) oa[d] += s[j] * (double)vr[d];
            }
            double delta = 0.0;
            for (int d = 0; d < D; ++d) delta += oa[d] * (double)go[d];
            for (long j = 0; j < ntot; ++j) {
                double pj = s[j];
                if (pj == 0.0) continue;
                int first = j < n1;
                long r = first ? (c0 + j) : (e0 + (j - n1));
                const float *kr = (first ? k1 : k2) + (r * Hkv + hk) * D;
                const float *vr = (first ? v1 : v2) + (r * Hkv + hk) * D;
                double *dkr = (first ? dk1 + j * D : dk2 + (j - n1) * D);
                double *dvr = (first ? dv1 + j * D : dv2 + (j - n1) * D);
                double dp = 0.0;
                for (int d = 0; d < D; ++d) dp += (double)go[d] * (double)vr[d];
                double ds = pj * (dp - delta) * scale;
                for (int d = 0; d < D; ++d) {
                    dvr[d] += pj * (double)go[d];
                    dkr[d] += ds * (double)qr[d];
                    dqa[d] += ds * (double)kr[d];
                }
            }
            for (int d = 0; d < D; ++d) dqr[d] = (float)dqa[d];
        }
    }
}

int duo_ref_bwd(const float *q1, const float *k1, const float *v1, const int *cu_q1,
                const int *cu_k1, const float *q2, const float *k2, const float *v2,
                const int *pos_q2, const int *pos_k2, const int *cu_q2, const int *cu_k2,
                int nseq, int Hq, int Hkv, int D, float scale_f,
                const float *do1, const float *do2,
                float *dq1, float *dk1, float *dv1, float *dq2, float *dk2, float *dv2)
{
    if (Hq % Hkv) return -1;
    double scale = (double)scale_f;
    long maxk = 0;
    for (int b = 0; b < nseq; ++b) {
        long n = (cu_k1[b + 1] - cu_k1[b]) + (cu_k2[b + 1] - cu_k2[b]);
        if (n > maxk) maxk = n;
    }
    int fail = 0;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int b = 0; b < nseq; ++b) {
        for (int hk = 0; hk < Hkv; ++hk) {
            long lq1 = cu_q1[b + 1] - cu_q1[b], lk1 = cu_k1[b + 1] - cu_k1[b];
            long lk2 = cu_k2[b + 1] - cu_k2[b];
            double *s = (double *)malloc(sizeof(double) * (size_t)(maxk + 1));
            double *acc = (double *)malloc(sizeof(double) * (size_t)(2 * D));
            double *a1 = (double *)calloc((size_t)(2 * lk1 * D + 1), sizeof(double));
            double *a2 = (double *)calloc((size_t)(2 * lk2 * D + 1), sizeof(double));
            if (!s || !acc || !a1 || !a2) { fail = 1; free(s); free(acc); free(a1); free(a2); continue; }
            double *gk1 = a1, *gv1 = a1 + lk1 * D, *gk2 = a2, *gv2 = a2 + lk2 * D;
            stream_bwd(q1, do1, cu_q1[b], cu_q1[b + 1], NULL, lk1 - lq1, k1, v1, cu_k1[b], lk1,
                       NULL, NULL, NULL, 0, 0, 0, Hq, Hkv, D, hk, scale, dq1, gk1, gv1, gk2, gv2, s, acc);
            stream_bwd(q2, do2, cu_q2[b], cu_q2[b + 1], pos_q2, 0, k1, v1, cu_k1[b], lk1,
                       k2, v2, pos_k2, cu_k2[b], lk2, 1, Hq, Hkv, D, hk, scale, dq2, gk1, gv1, gk2, gv2, s, acc);
            for (long j = 0; j < lk1; ++j)
                for (int d = 0; d < D; ++d) {
                    dk1[((cu_k1[b] + j) * Hkv + hk) * D + d] = (float)gk1[j * D + d];
                    dv1[((cu_k1[b] + j) * Hkv + hk) * D + d] = (float)gv1[j * D + d];
                }
            for (long j = 0; j < lk2; ++j)
                for (int d = 0; d < D; ++d) {
                    dk2[((cu_k2[b] + j) * Hkv + hk) * D + d] = (float)gk2[j * D + d];
                    dv2[((cu_k2[b] + j) * Hkv + hk) * D + d] = (float)gv2[j * D + d];
                }
            free(s); free(acc); free(a1); free(a2);
        }
    }
    return fail ? -2 : 0;
}

/* Hard-token index build: row-major order of True entries
 * (tah/model/tah_model.py:114-117, :163-167).  idx[r] = column of r-th True,
 * cu[b] = number of True entries in rows < b. */
int duo_ref_hard_index(const unsigned char *mask, int B, int S, int *idx, int *cu)
{
    int n = 0;
    for (int b = 0; b < B; ++b) {
        cu[b] = n;
        for (int s = 0; s < S; ++s)
            if (mask[(long)b * S + s]) idx[n++] = s;
    }
    cu[B] = n;
    return n;
}

/*
 * CPU restatement (plain C, OpenMP over independent recurrences) of the gated delta rule.
 *
 * TEST INFRASTRUCTURE ONLY: nothing in the shipped package links or loads this file.
 * It exists so that parity can be checked at the full benchmark sizes in seconds, where
 * the torch token loop of oracle/gdn_oracle.py would take minutes.
 *
 * Follows the operator the reference layer calls at
 *   lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:197-222
 * (third-party `fla`, un-vendored, version unpinned), restated from its published
 * recurrence; state layout [N, H, K, V] and the token loop follow the reference's naive
 * ops (.../linear_attention/op.py:36-44).  cu_seqlens convention:
 *   lm_engine/modeling_utils/sequence_packing.py:18-22 (int32, leading 0).
 *
 * PARITY UNPINNED at the `fla` boundary (no reference fixture exists for this path);
 * pinned instead against oracle/gdn_oracle.py and closed forms by tests/test_oracle_c.py.
 *
 * Per (sequence n, head h), token t:
 *     q^ = (q / sqrt(|q|^2 + 1e-6) if l2norm else q) * scale ;  k^ likewise without scale
 *     S <- exp(g) S ;  r = beta (v - S^T k^) ;  S <- S + k^ r^T ;  o = S^T q^
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define GDN_ORACLE_EPS 1e-6

#define DEFINE_CHAIN(NAME, REAL)                                                                        \
    static void NAME(const float *q, const float *k, const float *v, const float *g, const float *beta, \
                     const float *h0, float *o, float *ht, long t0, long t1, long tok_stride_qk,        \
                     long tok_stride_v, long tok_stride_s, int K, int V, float scale, int l2norm,      \
                     REAL *S, REAL *qh, REAL *kh, REAL *sk, REAL *acc)                                  \
    {                                                                                                   \
        for (long i = 0; i < (long)K * V; i++) S[i] = h0 ? (REAL)h0[i] : (REAL)0;                       \
        for (long t = t0; t < t1; t++) {                                                                \
            const float *qt = q + t * tok_stride_qk, *kt = k + t * tok_stride_qk;                       \
            const float *vt = v + t * tok_stride_v;                                                     \
            float *ot = o + t * tok_stride_v;                                                           \
            REAL qn = 1, kn = 1;                                                                        \
            if (l2norm) {                                                                               \
                REAL sq = 0, sn = 0;                                                                    \
                for (int d = 0; d < K; d++) { sq += (REAL)qt[d] * qt[d]; sn += (REAL)kt[d] * kt[d]; }   \
                qn = 1 / sqrt(sq + (REAL)GDN_ORACLE_EPS);                                               \
                kn = 1 / sqrt(sn + (REAL)GDN_ORACLE_EPS);                                               \
            }                                                                                           \
            for (int d = 0; d < K; d++) { qh[d] = (REAL)qt[d] * qn * (REAL)scale; kh[d] = (REAL)kt[d] * kn; } \
            REAL eg = g ? exp((REAL)g[t * tok_stride_s]) : (REAL)1;                                     \
            REAL b = beta ? (REAL)beta[t * tok_stride_s] : (REAL)1;                                     \
            for (int j = 0; j < V; j++) { sk[j] = 0; acc[j] = 0; }                                      \
            for (int d = 0; d < K; d++) {                                                               \
                REAL *Sd = S + (long)d * V;                                                             \
                REAL kd = kh[d];                                                                        \
                for (int j = 0; j < V; j++) { Sd[j] *= eg; sk[j] += Sd[j] * kd; }                       \
            }                                                                                           \
            for (int j = 0; j < V; j++) sk[j] = b * ((REAL)vt[j] - sk[j]); /* sk now holds r */         \
            for (int d = 0; d < K; d++) {                                                               \
                REAL *Sd = S + (long)d * V;                                                             \
                REAL kd = kh[d], qd = qh[d];                                                            \
                for (int j = 0; j < V; j++) { Sd[j] += kd * sk[j]; acc[j] += Sd[j] * qd; }              \
            }                                                                                           \
            for (int j = 0; j < V; j++) ot[j] = (float)acc[j];                                          \
        }                                                                                               \
        if (ht) for (long i = 0; i < (long)K * V; i++) ht[i] = (float)S[i];                             \
    }

DEFINE_CHAIN(chain_f32, float)
DEFINE_CHAIN(chain_f64, double)

/*
 * q, k: [B, T, H, K] fp32 contiguous; v, o: [B, T, H, V]; g, beta: [B, T, H] or NULL;
 * h0, ht: [N, H, K, V] or NULL; cu_seqlens: host int32 [N+1] or NULL (then N == B).
 * Returns 0, or -1 on inconsistent arguments.
 */
int gdn_oracle_recurrent(const float *q, const float *k, const float *v, const float *g, const float *beta,
                         const float *h0, float *o, float *ht, const int32_t *cu_seqlens, int B, int T, int H,
                         int K, int V, int N, float scale, int l2norm, int f64_state)
{
    if (cu_seqlens && B != 1) return -1;
    if (!cu_seqlens && N != B) return -1;
    long work = (long)N * H;
    int bad = 0;
#pragma omp parallel
    {
        void *S = malloc((size_t)K * V * sizeof(double));
        void *qh = malloc((size_t)K * sizeof(double));
        void *kh = malloc((size_t)K * sizeof(double));
        void *sk = malloc((size_t)V * sizeof(double));
        void *acc = malloc((size_t)V * sizeof(double));
        if (!S || !qh || !kh || !sk || !acc) {
#pragma omp atomic write
            bad = 1;
        } else {
#pragma omp for schedule(dynamic, 1)
            for (long w = 0; w < work; w++) {
                int n = (int)(w / H), h = (int)(w % H);
                long b = cu_seqlens ? 0 : n;
                long t0 = cu_seqlens ? cu_seqlens[n] : 0;
                long t1 = cu_seqlens ? cu_seqlens[n + 1] : T;
                const float *qb = q + (b * T * H + h) * (long)K;
                const float *kb = k + (b * T * H + h) * (long)K;
                const float *vb = v + (b * T * H + h) * (long)V;
                float *ob = o + (b * T * H + h) * (long)V;
                const float *gb = g ? g + b * T * H + h : NULL;
                const float *bb = beta ? beta + b * T * H + h : NULL;
                const float *h0b = h0 ? h0 + ((long)n * H + h) * K * V : NULL;
                float *htb = ht ? ht + ((long)n * H + h) * K * V : NULL;
                if (f64_state)
                    chain_f64(qb, kb, vb, gb, bb, h0b, ob, htb, t0, t1, (long)H * K, (long)H * V, H, K, V, scale,
                              l2norm, (double *)S, (double *)qh, (double *)kh, (double *)sk, (double *)acc);
                else
                    chain_f32(qb, kb, vb, gb, bb, h0b, ob, htb, t0, t1, (long)H * K, (long)H * V, H, K, V, scale,
                              l2norm, (float *)S, (float *)qh, (float *)kh, (float *)sk, (float *)acc);
            }
        }
        free(S);
        free(qh);
        free(kh);
        free(sk);
        free(acc);
    }
    return bad ? -2 : 0;
}

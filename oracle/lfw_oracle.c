/*
 * CPU oracle (plain C, double precision) for the decay-rule recurrence.
 *
 * TEST INFRASTRUCTURE ONLY.  The shipped library never links or loads this file; it
 * is built by oracle/build.py into oracle/_build/ and loaded by tests, the smoke
 * check and the CPU-baseline leg of the benchmark.
 *
 * What each function follows in the reference tree:
 *   lfw_oracle_forward   t2fw/torch.py:21-31 (recurrence; output from the updated
 *                        state; final state returned), element loop as in
 *                        t2fw/csrc/lfw_kernel.cu:43-57 + the output contraction of
 *                        t2fw/csrc/lfw.cpp:45
 *   lfw_oracle_backward  t2fw/csrc/lfw_kernel.cu:85-100 (reverse scan of the state
 *                        gradient) + t2fw/csrc/lfw.cpp:84-93 (six contractions)
 *
 * Pinning: tests/test_oracle_lfw.py checks both against the torch restatement's
 * autograd, closed forms, the brute-force unrolled sum and finite differences.
 *
 * Layout: x,f,g_out,out,d_x,d_f [B,T,D]; q,k,fk,d_q,d_k,d_fk [B,T,K];
 * s0,next_state,g_state,d_s0 [B,D,K]; all dense row-major doubles.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

int lfw_oracle_forward(const double *x, const double *f, const double *q,
                       const double *k, const double *fk, const double *s0,
                       double *out, double *next_state,
                       int64_t B, int64_t T, int64_t D, int64_t K)
{
    int64_t b;
#pragma omp parallel for schedule(dynamic, 1)
    for (b = 0; b < B; ++b) {
        double *S = next_state + b * D * K;   /* running state, ends as S_{T-1} */
        memcpy(S, s0 + b * D * K, sizeof(double) * (size_t)(D * K));
        for (int64_t t = 0; t < T; ++t) {
            const double *xt = x + (b * T + t) * D, *ft = f + (b * T + t) * D;
            const double *qt = q + (b * T + t) * K, *kt = k + (b * T + t) * K;
            const double *gt = fk + (b * T + t) * K;
            double *ot = out + (b * T + t) * D;
            for (int64_t d = 0; d < D; ++d) {
                double acc = 0.0;
                for (int64_t c = 0; c < K; ++c) {
                    double s = S[d * K + c] * (ft[d] * gt[c]) + xt[d] * kt[c];
                    S[d * K + c] = s;
                    acc += s * qt[c];
                }
                ot[d] = acc;
            }
        }
    }
    return 0;
}

int lfw_oracle_backward(const double *g_out, const double *g_state,
                        const double *x, const double *f, const double *q,
                        const double *k, const double *fk, const double *s0,
                        double *d_x, double *d_f, double *d_q, double *d_k,
                        double *d_fk, double *d_s0,
                        int64_t B, int64_t T, int64_t D, int64_t K)
{
    int64_t b;
    int failed = 0;
#pragma omp parallel for schedule(dynamic, 1)
    for (b = 0; b < B; ++b) {
        const int64_t DK = D * K;
        /* all states S_{-1}=s0, S_0 .. S_{T-1}  (the reference keeps them too) */
        double *S = (double *)malloc(sizeof(double) * (size_t)((T + 1) * DK));
        if (!S) { failed = 1; continue; }
        memcpy(S, s0 + b * DK, sizeof(double) * (size_t)DK);
        for (int64_t t = 0; t < T; ++t) {
            const double *xt = x + (b * T + t) * D, *ft = f + (b * T + t) * D;
            const double *kt = k + (b * T + t) * K, *gt = fk + (b * T + t) * K;
            const double *Sp = S + t * DK;
            double *Sn = S + (t + 1) * DK;
            for (int64_t d = 0; d < D; ++d)
                for (int64_t c = 0; c < K; ++c)
                    Sn[d * K + c] = Sp[d * K + c] * (ft[d] * gt[c]) + xt[d] * kt[c];
        }
        double *G = d_s0 + b * DK;
        memcpy(G, g_state + b * DK, sizeof(double) * (size_t)DK);
        for (int64_t t = T - 1; t >= 0; --t) {
            const double *xt = x + (b * T + t) * D, *ft = f + (b * T + t) * D;
            const double *qt = q + (b * T + t) * K, *kt = k + (b * T + t) * K;
            const double *gt = fk + (b * T + t) * K, *go = g_out + (b * T + t) * D;
            const double *Sp = S + t * DK, *Sn = S + (t + 1) * DK;
            double *dxt = d_x + (b * T + t) * D, *dft = d_f + (b * T + t) * D;
            double *dqt = d_q + (b * T + t) * K, *dkt = d_k + (b * T + t) * K;
            double *dgt = d_fk + (b * T + t) * K;
            for (int64_t c = 0; c < K; ++c) { dqt[c] = 0; dkt[c] = 0; dgt[c] = 0; }
            for (int64_t d = 0; d < D; ++d) {
                double ax = 0.0, af = 0.0;
                for (int64_t c = 0; c < K; ++c) {
                    double g = go[d] * qt[c] + G[d * K + c];  /* lfw_kernel.cu:89 */
                    double h = g * Sp[d * K + c];             /* lfw.cpp:89-90 */
                    dqt[c] += go[d] * Sn[d * K + c];          /* lfw.cpp:84 */
                    ax += g * kt[c];                          /* lfw.cpp:85 */
                    dkt[c] += g * xt[d];                      /* lfw.cpp:86 */
                    af += h * gt[c];                          /* lfw.cpp:92 */
                    dgt[c] += h * ft[d];                      /* lfw.cpp:93 */
                    G[d * K + c] = g * (ft[d] * gt[c]);       /* lfw_kernel.cu:93 */
                }
                dxt[d] = ax;
                dft[d] = af;
            }
        }
        free(S);
    }
    return failed;
}

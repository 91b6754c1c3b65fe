/*
 * flare_oracle.c — plain-C CPU restatement of the FLARE hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  It is compiled into oracle/libflare_oracle.so and called
 * from tests/, the smoke check and the benchmark's cpu_baseline leg as a CHECKER; the
 * product library never links, loads or calls it.
 *
 * Contiguous row-major fp32 in and out, double accumulation inside, so that it is an
 * independent second opinion on the torch restatement in flare_oracle.py.
 *
 *   oracle_mixer    README.md:39-52 of the reference (two softmax-attention calls),
 *                   spelled out as pdebench/models/flare.py:142-150 does
 *   oracle_causal   causal restriction of the mixer, token recurrence in the shape of
 *                   lra/models/triton/causal_linear.py:317-336 (the reference has no
 *                   causal-FLARE code of its own)
 *   oracle_triple   lra/models/backends.py:1285-1292 (einsum pair), feature map
 *                   lra/models/kernels.py:23-24
 *
 * Pinning: see the header of flare_oracle.py; tests/test_oracle.py checks this file
 * against the torch restatement, closed forms and brute force.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* q [H,M,D] shared over batch; k,v,y [B,H,N,D]; z [B,H,M,D].  key_mask [B,N] or NULL. */
int oracle_mixer(const float* q, const float* k, const float* v, const uint8_t* key_mask,
                 float* y, float* z, int B, int H, int N, int M, int D, float scale)
{
    int bh;
#pragma omp parallel for schedule(dynamic)
    for (bh = 0; bh < B * H; ++bh) {
        int b = bh / H, h = bh % H;
        const float* qh = q + (size_t)h * M * D;
        const float* kb = k + (size_t)bh * N * D;
        const float* vb = v + (size_t)bh * N * D;
        float* yb = y + (size_t)bh * N * D;
        float* zb = z + (size_t)bh * M * D;
        const uint8_t* mk = key_mask ? key_mask + (size_t)b * N : NULL;
        double* zz = (double*)calloc((size_t)M * D, sizeof(double));
        double* sc = (double*)malloc((size_t)(N > M ? N : M) * sizeof(double));
        for (int m = 0; m < M; ++m) {
            double mx = -INFINITY;
            for (int n = 0; n < N; ++n) {
                double s = 0.0;
                for (int d = 0; d < D; ++d) s += (double)qh[m * D + d] * kb[(size_t)n * D + d];
                s *= scale;
                if (mk && !mk[n]) s = -INFINITY;
                sc[n] = s;
                if (s > mx) mx = s;
            }
            double tot = 0.0;
            for (int n = 0; n < N; ++n) {
                if (sc[n] == -INFINITY) continue;
                double e = exp(sc[n] - mx);
                tot += e;
                for (int d = 0; d < D; ++d) zz[m * D + d] += e * vb[(size_t)n * D + d];
            }
            for (int d = 0; d < D; ++d) {
                zz[m * D + d] = tot > 0.0 ? zz[m * D + d] / tot : 0.0;
                zb[m * D + d] = (float)zz[m * D + d];
            }
        }
        for (int n = 0; n < N; ++n) {
            double mx = -INFINITY, tot = 0.0;
            for (int m = 0; m < M; ++m) {
                double s = 0.0;
                for (int d = 0; d < D; ++d) s += (double)qh[m * D + d] * kb[(size_t)n * D + d];
                sc[m] = s * scale;
                if (sc[m] > mx) mx = sc[m];
            }
            for (int m = 0; m < M; ++m) { sc[m] = exp(sc[m] - mx); tot += sc[m]; }
            for (int d = 0; d < D; ++d) {
                double acc = 0.0;
                for (int m = 0; m < M; ++m) acc += sc[m] * zz[m * D + d];
                yb[(size_t)n * D + d] = (mk && !mk[n]) ? 0.0f : (float)(acc / tot);
            }
        }
        free(zz);
        free(sc);
    }
    return 0;
}

/* Token recurrence.  State mu,den [B,H,M], num [B,H,M,D] (double) is advanced in place;
 * a fresh state is mu = -INFINITY, den = num = 0. */
int oracle_causal(const float* q, const float* k, const float* v, float* y, double* mu,
                  double* den, double* num, int B, int H, int N, int M, int D, float scale)
{
    int bh;
#pragma omp parallel for schedule(dynamic)
    for (bh = 0; bh < B * H; ++bh) {
        int h = bh % H;
        const float* qh = q + (size_t)h * M * D;
        double* mub = mu + (size_t)bh * M;
        double* deb = den + (size_t)bh * M;
        double* nub = num + (size_t)bh * M * D;
        double* sg = (double*)malloc((size_t)M * sizeof(double));
        for (int t = 0; t < N; ++t) {
            const float* kt = k + ((size_t)bh * N + t) * D;
            const float* vt = v + ((size_t)bh * N + t) * D;
            float* yt = y + ((size_t)bh * N + t) * D;
            double smax = -INFINITY;
            for (int m = 0; m < M; ++m) {
                double s = 0.0;
                for (int d = 0; d < D; ++d) s += (double)qh[m * D + d] * kt[d];
                s *= scale;
                sg[m] = s;
                if (s > smax) smax = s;
                double mn = mub[m] > s ? mub[m] : s;
                double a = (mub[m] == -INFINITY) ? 0.0 : exp(mub[m] - mn);
                double p = exp(s - mn);
                deb[m] = a * deb[m] + p;
                for (int d = 0; d < D; ++d) nub[m * D + d] = a * nub[m * D + d] + p * vt[d];
                mub[m] = mn;
            }
            double tot = 0.0;
            for (int m = 0; m < M; ++m) { sg[m] = exp(sg[m] - smax); tot += sg[m]; }
            for (int d = 0; d < D; ++d) {
                double acc = 0.0;
                for (int m = 0; m < M; ++m) acc += sg[m] * nub[m * D + d] / deb[m];
                yt[d] = (float)(acc / tot);
            }
        }
        free(sg);
    }
    return 0;
}

static inline double feat(double x, int feature_map)
{
    if (!feature_map) return x;
    return x > 0.0 ? x + 1.0 : exp(x); /* elu(x) + 1 */
}

/* q1,q2,k1,k2 [B,H,N,Dq]; v,out [B,H,N,Dv]; state [B,H,Dq,Dv,Dq] (index i,j,k). */
int oracle_triple(const float* q1, const float* q2, const float* k1, const float* k2,
                  const float* v, float* state, float* out, int B, int H, int N, int Dq, int Dv,
                  int feature_map, int normalize)
{
    int bh;
#pragma omp parallel for schedule(dynamic)
    for (bh = 0; bh < B * H; ++bh) {
        size_t qo = (size_t)bh * N * Dq, vo = (size_t)bh * N * Dv;
        size_t ns = (size_t)Dq * Dv * Dq;
        double* st = (double*)calloc(ns, sizeof(double));
        double* kk = (double*)calloc((size_t)Dq * Dq, sizeof(double));
        for (int n = 0; n < N; ++n)
            for (int i = 0; i < Dq; ++i) {
                double a = feat(k1[qo + (size_t)n * Dq + i], feature_map);
                for (int kx = 0; kx < Dq; ++kx) {
                    double c = feat(k2[qo + (size_t)n * Dq + kx], feature_map);
                    kk[i * Dq + kx] += a * c;
                    for (int j = 0; j < Dv; ++j)
                        st[((size_t)i * Dv + j) * Dq + kx] += a * c * v[vo + (size_t)n * Dv + j];
                }
            }
        for (size_t e = 0; e < ns; ++e) { st[e] /= N; state[bh * ns + e] = (float)st[e]; }
        for (int e = 0; e < Dq * Dq; ++e) kk[e] /= N;
        for (int n = 0; n < N; ++n) {
            double dn = 0.0;
            for (int i = 0; i < Dq; ++i)
                for (int kx = 0; kx < Dq; ++kx)
                    dn += feat(q1[qo + (size_t)n * Dq + i], feature_map) * kk[i * Dq + kx] *
                          feat(q2[qo + (size_t)n * Dq + kx], feature_map);
            for (int j = 0; j < Dv; ++j) {
                double acc = 0.0;
                for (int i = 0; i < Dq; ++i) {
                    double a = feat(q1[qo + (size_t)n * Dq + i], feature_map);
                    for (int kx = 0; kx < Dq; ++kx)
                        acc += a * st[((size_t)i * Dv + j) * Dq + kx] *
                               feat(q2[qo + (size_t)n * Dq + kx], feature_map);
                }
                out[vo + (size_t)n * Dv + j] = (float)(normalize ? acc / dn : acc);
            }
        }
        free(st);
        free(kk);
    }
    return 0;
}

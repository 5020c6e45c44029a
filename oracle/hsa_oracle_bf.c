/*
 * Brute-force C restatement of the hierarchical sparse attention forward path.
 *
 * TEST INFRASTRUCTURE ONLY: linked by nothing in the shipped package; loaded by
 * the test-suite (and the benchmark's CPU-baseline leg) through ctypes as an
 * independent check of oracle/hsa_oracle.py and of the HIP kernels.
 *
 * Every routine walks the slots one by one in double precision, the way the
 * reference kernel enumerates them, with no vectorised gather:
 *   attention     hierarchical_attention/ops/triton/sparse_attn.py:8-179
 *   parent build  hierarchical_attention/ops/triton/build_parents.py:8-99
 *   topology      hierarchical_attention_project/Hierarchical_Attention_Triton_Test.py:40-104
 *                 (forward climb) and hierarchical_attention/ops/topology.py:64-122
 *                 (sibling leaf ranges), the latter by explicit descent to the leaves.
 *
 * Build: gcc -O2 -fopenmp -shared -fPIC -o libhsa_oracle_bf.so hsa_oracle_bf.c -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

/* Q [B,N,H,D]; K,V [B,M,H,D]; idx [N,L]; mask [N,L] or NULL (NULL = non-causal).
 * out [B,N,H,D]; weights [B,N,H,2R+1+L] or NULL. */
void hsa_oracle_attention(const float *Q, const float *K, const float *V, const int32_t *idx,
                          const uint8_t *mask, float *out, float *weights, int B, int N, int M,
                          int H, int D, int L, int R)
{
    const int S = 2 * R + 1 + L;
    const double scale = 1.0 / sqrt((double)D);
    const int causal = mask != NULL;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
        for (int n = 0; n < N; ++n) {
            double *s = (double *)malloc(sizeof(double) * S);
            int *row = (int *)malloc(sizeof(int) * S);
            for (int h = 0; h < H; ++h) {
                const float *q = Q + (((size_t)b * N + n) * H + h) * D;
                for (int w = 0; w < 2 * R + 1; ++w) {
                    int j = n + w - R;
                    int live = j >= 0 && j < N && (!causal || j <= n);
                    row[w] = live ? j : -1;
                }
                for (int l = 0; l < L; ++l) {
                    int m = idx[(size_t)n * L + l];
                    int live = m != -1 && (!causal || !mask[(size_t)n * L + l]);
                    row[2 * R + 1 + l] = live ? m : -1;
                }
                double mx = -INFINITY;
                for (int t = 0; t < S; ++t) {
                    if (row[t] < 0) { s[t] = -INFINITY; continue; }
                    const float *k = K + (((size_t)b * M + row[t]) * H + h) * D;
                    double acc = 0.0;
                    for (int d = 0; d < D; ++d) acc += (double)q[d] * (double)k[d];
                    s[t] = acc * scale;
                    if (s[t] > mx) mx = s[t];
                }
                double den = 0.0;
                for (int t = 0; t < S; ++t) {
                    s[t] = row[t] < 0 ? 0.0 : exp(s[t] - mx);
                    den += s[t];
                }
                if (den < 1.0e-5) den = 1.0e-5;
                float *o = out + (((size_t)b * N + n) * H + h) * D;
                for (int d = 0; d < D; ++d) {
                    double acc = 0.0;
                    for (int t = 0; t < S; ++t)
                        if (row[t] >= 0)
                            acc += s[t] / den * (double)V[(((size_t)b * M + row[t]) * H + h) * D + d];
                    o[d] = (float)acc;
                }
                if (weights) {
                    float *wp = weights + (((size_t)b * N + n) * H + h) * S;
                    for (int t = 0; t < S; ++t) wp[t] = (float)(s[t] / den);
                }
            }
            free(s);
            free(row);
        }
}

/* qp,kp,vp [B,P,H,D]; kc,vc [B,2P,H,D]; out [B,P,H,D]; w [B,P,H,3] or NULL. */
void hsa_oracle_build_parents(const float *qp, const float *kp, const float *vp, const float *kc,
                              const float *vc, float *out, float *w, int B, int P, int H, int D)
{
    const double scale = 1.0 / sqrt((double)D);
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
        for (int i = 0; i < P; ++i)
            for (int h = 0; h < H; ++h) {
                size_t po = (((size_t)b * P + i) * H + h) * D;
                size_t c0 = (((size_t)b * 2 * P + 2 * i) * H + h) * D;
                size_t c1 = (((size_t)b * 2 * P + 2 * i + 1) * H + h) * D;
                double s[3] = {0, 0, 0};
                for (int d = 0; d < D; ++d) {
                    s[0] += (double)qp[po + d] * kp[po + d];
                    s[1] += (double)qp[po + d] * kc[c0 + d];
                    s[2] += (double)qp[po + d] * kc[c1 + d];
                }
                double mx = -INFINITY;
                for (int t = 0; t < 3; ++t) { s[t] *= scale; if (s[t] > mx) mx = s[t]; }
                double den = 1e-9;
                for (int t = 0; t < 3; ++t) { s[t] = exp(s[t] - mx); den += s[t]; }
                for (int t = 0; t < 3; ++t) s[t] /= den;
                for (int d = 0; d < D; ++d)
                    out[po + d] = (float)(s[0] * vp[po + d] + s[1] * vc[c0 + d] + s[2] * vc[c1 + d]);
                if (w) {
                    size_t wo = (((size_t)b * P + i) * H + h) * 3;
                    w[wo] = (float)s[0]; w[wo + 1] = (float)s[1]; w[wo + 2] = (float)s[2];
                }
            }
}

/* leftmost / rightmost+1 leaf under node i, by walking children. Level-l nodes
 * start at first[l]; children of first[l]+j are first[l-1]+2j and +2j+1. */
static void leaf_span(int node, int N, int *lo, int *hi, int *level)
{
    int start = 0, count = N, lvl = 0;
    while (node >= start + count) { start += count; count /= 2; ++lvl; }
    int j = node - start;
    *level = lvl;
    *lo = j << lvl;
    *hi = (j + 1) << lvl;
    /* descend explicitly to confirm: leftmost leaf */
    int a = node, s = start, c = count, L = lvl;
    while (L > 0) { int jj = a - s; c *= 2; s -= c; a = s + 2 * jj; --L; }
    *lo = a;
    a = node; s = start; c = count; L = lvl;
    while (L > 0) { int jj = a - s; c *= 2; s -= c; a = s + 2 * jj + 1; --L; }
    *hi = a + 1;
}

/* idx [N,L] int32, mask [N,L] uint8, gather [2N-1,3] int32. */
void hsa_oracle_topology(int N, int causal, int32_t *idx, uint8_t *mask, int32_t *gather)
{
    int L = 0;
    while ((1 << L) < N) ++L;
    const int total = 2 * N - 1, max_valid = total - 2;
    for (int n = 0; n < N; ++n) {
        for (int l = 0; l < L; ++l) { idx[(size_t)n * L + l] = -1; mask[(size_t)n * L + l] = 0; }
        int cur = n;
        for (int l = 0; l < L; ++l) {
            int nxt, pair;
            if (l == 0) { nxt = cur ^ 1; pair = cur; }
            else { pair = cur / 2 + N; nxt = pair ^ 1; }
            if (nxt > max_valid) break;
            if (causal && pair < nxt) mask[(size_t)n * L + l] = 1;
            idx[(size_t)n * L + l] = nxt;
            cur = nxt;
        }
    }
    for (int i = 0; i < total; ++i) {
        int sib = i ^ 1;
        if (sib > total - 1) sib = total - 1;
        int take = sib != i && (!causal || sib > i);
        if (!take) { gather[3 * i] = gather[3 * i + 1] = gather[3 * i + 2] = -1; continue; }
        int lo, hi, lv, mylo, myhi, mylv;
        leaf_span(sib, N, &lo, &hi, &lv);
        leaf_span(i, N, &mylo, &myhi, &mylv);
        gather[3 * i] = lo; gather[3 * i + 1] = hi; gather[3 * i + 2] = mylv;
    }
}

/*
 * TEST INFRASTRUCTURE -- CPU oracle, never a product path.
 *
 * Plain-C restatement of DA-Transformer's DAG training operators, written from the
 * recurrences, independent of torch.  Used by the tests to pin the torch restatement
 * (oracle/torch_native.py) and as a checker for the HIP kernels.  Nothing under the
 * shipped package links or loads this file.
 *
 * Conventions (same as the reference's torch-native functions, square links):
 *   match[b][t][j]  log P(target t | node j)            [B,T,L]
 *   links[b][i][j]  log P(i -> j), -inf when no edge    [B,L,L]
 *   out_len[b]=L_b, tgt_len[b]=T_b
 *
 * Reference lines restated:
 *   dagref_loss_f64        fs_plugins/custom_ops/dag_loss.py:259-300 (alpha sweep, read-out at
 *                          (T_b-1, L_b-1)); beta sweep as fs_plugins/custom_ops/dag_loss.cu:178-274
 *   dagref_loss_grad_f64   fs_plugins/custom_ops/dag_loss.cu:378-401 (grad of match),
 *                          :432-485 (grad of links); equal to autograd through dag_loss.py:259-300
 *   dagref_align_f32       fs_plugins/custom_ops/dag_loss.py:253-257, 303-353 (fp32, add then max
 *                          then add; lowest predecessor index wins ties) with the backtrack of
 *                          fs_plugins/custom_ops/dag_best_alignment.cu:170-189
 *   dagref_lsg_f64         fs_plugins/custom_ops/dag_loss.py:355-359
 *   dagref_lsg_bwd_f64     fs_plugins/custom_ops/dag_loss.py:216-231 (softmax Jacobian + scatter)
 *
 * Pins: tests/test_oracle_*.py check these against brute-force path enumeration, closed
 * forms and the torch restatement.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define NEG_INF (-INFINITY)

static double lse_pair_sum(const double *v, int n) {
    /* log sum exp of v[0..n); -inf if every term is -inf */
    double top = NEG_INF;
    for (int k = 0; k < n; ++k) if (v[k] > top) top = v[k];
    if (top == NEG_INF) return NEG_INF;
    double s = 0.0;
    for (int k = 0; k < n; ++k) s += exp(v[k] - top);
    return top + log(s);
}

/* alpha[b][t][j], beta[b][t][j] (both [B,T,L], filled with -inf outside the DP), loss[b].
 * Returns 0. */
int dagref_loss_f64(const double *match, const double *links, const int64_t *out_len,
                    const int64_t *tgt_len, int B, int T, int L,
                    double *alpha, double *beta, double *loss) {
    /* samples are independent: one thread per sample (the arithmetic of a sample is unchanged) */
#pragma omp parallel for schedule(dynamic, 1)
    for (int b = 0; b < B; ++b) {
        const double *m = match + (size_t)b * T * L;
        const double *e = links + (size_t)b * L * L;
        double *a = alpha + (size_t)b * T * L;
        double *bt = beta + (size_t)b * T * L;
        int Lb = (int)out_len[b], Tb = (int)tgt_len[b];
        for (size_t k = 0; k < (size_t)T * L; ++k) { a[k] = NEG_INF; bt[k] = NEG_INF; }
        if (Tb < 1 || Lb < 1 || Tb > T || Lb > L) { loss[b] = NEG_INF; continue; }
        double *tmp = (double *)malloc(sizeof(double) * (size_t)L);
        a[0] = m[0];
        for (int t = 1; t < Tb; ++t)
            for (int j = 0; j < Lb; ++j) {
                int n = 0;
                for (int i = 0; i < j; ++i) tmp[n++] = a[(size_t)(t - 1) * L + i] + e[(size_t)i * L + j];
                a[(size_t)t * L + j] = lse_pair_sum(tmp, n) + m[(size_t)t * L + j];
            }
        loss[b] = a[(size_t)(Tb - 1) * L + (Lb - 1)];
        bt[(size_t)(Tb - 1) * L + (Lb - 1)] = m[(size_t)(Tb - 1) * L + (Lb - 1)];
        for (int t = Tb - 2; t >= 0; --t)
            for (int i = 0; i < Lb; ++i) {
                int n = 0;
                for (int j = i + 1; j < Lb; ++j) tmp[n++] = e[(size_t)i * L + j] + bt[(size_t)(t + 1) * L + j];
                bt[(size_t)t * L + i] = lse_pair_sum(tmp, n) + m[(size_t)t * L + i];
            }
        free(tmp);
    }
    return 0;
}

/* grad_match [B,T,L], grad_links [B,L,L] (square) for upstream gradient g[b].
 * Infeasible samples (Z = -inf) get all-zero gradients. */
int dagref_loss_grad_f64(const double *match, const double *links, const int64_t *out_len,
                         const int64_t *tgt_len, const double *g, int B, int T, int L,
                         const double *alpha, const double *beta,
                         double *grad_match, double *grad_links) {
    memset(grad_match, 0, sizeof(double) * (size_t)B * T * L);
    memset(grad_links, 0, sizeof(double) * (size_t)B * L * L);
#pragma omp parallel for schedule(dynamic, 1)
    for (int b = 0; b < B; ++b) {
        const double *m = match + (size_t)b * T * L;
        const double *e = links + (size_t)b * L * L;
        const double *a = alpha + (size_t)b * T * L;
        const double *bt = beta + (size_t)b * T * L;
        double *gm = grad_match + (size_t)b * T * L;
        double *gl = grad_links + (size_t)b * L * L;
        int Lb = (int)out_len[b], Tb = (int)tgt_len[b];
        if (Tb < 1 || Lb < 1 || Tb > T || Lb > L) continue;
        double Z = bt[0];
        if (isinf(Z) || isnan(Z)) continue;
        for (int t = 0; t < Tb; ++t)
            for (int j = 0; j < Lb; ++j) {
                double mv = m[(size_t)t * L + j];
                if (isinf(mv)) continue;
                gm[(size_t)t * L + j] = g[b] * exp(a[(size_t)t * L + j] + bt[(size_t)t * L + j] - mv - Z);
            }
        for (int i = 0; i < Lb; ++i)
            for (int j = i + 1; j < Lb; ++j) {
                double ev = e[(size_t)i * L + j];
                if (ev == NEG_INF) continue;
                double s = 0.0;
                for (int t = 0; t + 1 < Tb; ++t) {
                    double x = a[(size_t)t * L + i] + ev + bt[(size_t)(t + 1) * L + j] - Z;
                    if (x > NEG_INF) s += exp(x);
                }
                gl[(size_t)i * L + j] = g[b] * s;
            }
    }
    return 0;
}

/* Viterbi in fp32 with exactly two roundings per cell, lowest-index ties, then backtrack.
 * path[b][j] = t or -1 ([B,L] int64); score[b] = best score (may be NULL).  Samples with no
 * finite-score path, or with lengths outside 1<=T_b<=L_b, get an all -1 row. */
int dagref_align_f32(const float *match, const float *links, const int64_t *out_len,
                     const int64_t *tgt_len, int B, int T, int L,
                     int64_t *path, float *score) {
#pragma omp parallel for schedule(dynamic, 1)
    for (int b = 0; b < B; ++b) {
        const float *m = match + (size_t)b * T * L;
        const float *e = links + (size_t)b * L * L;
        int64_t *p = path + (size_t)b * L;
        int Lb = (int)out_len[b], Tb = (int)tgt_len[b];
        for (int j = 0; j < L; ++j) p[j] = -1;
        if (score) score[b] = NEG_INF;
        if (Tb < 1 || Lb < 1 || Tb > T || Lb > L || Tb > Lb) continue;
        float *cur = (float *)malloc(sizeof(float) * (size_t)L);
        float *nxt = (float *)malloc(sizeof(float) * (size_t)L);
        int32_t *back = (int32_t *)malloc(sizeof(int32_t) * (size_t)T * L);
        for (int j = 0; j < L; ++j) cur[j] = NEG_INF;
        cur[0] = m[0];
        for (int t = 1; t < Tb; ++t) {
            for (int j = 0; j < Lb; ++j) {
                float best = NEG_INF; int arg = 0;
                for (int i = 0; i < j; ++i) {
                    volatile float cand = cur[i] + e[(size_t)i * L + j]; /* rounded to fp32 */
                    if (cand > best) { best = cand; arg = i; }
                }
                volatile float cell = best + m[(size_t)t * L + j];
                nxt[j] = cell;
                back[(size_t)t * L + j] = arg;
            }
            for (int j = Lb; j < L; ++j) nxt[j] = NEG_INF;
            float *sw = cur; cur = nxt; nxt = sw;
        }
        float fin = cur[Lb - 1];
        if (score) score[b] = fin;
        if (fin > NEG_INF) {
            int j = Lb - 1;
            for (int t = Tb - 1; t >= 0; --t) {
                p[j] = t;
                if (t > 0) j = back[(size_t)t * L + j];
            }
        }
        free(cur); free(nxt); free(back);
    }
    return 0;
}

/* sel[r][s] = log_softmax(x[r][:])[idx[r][s]] for `rows` rows of V logits; lse[r] = log sum exp. */
int dagref_lsg_f64(const double *x, const int64_t *idx, int rows, int V, int S,
                   double *sel, double *lse) {
    for (int r = 0; r < rows; ++r) {
        double z = lse_pair_sum(x + (size_t)r * V, V);
        if (lse) lse[r] = z;
        for (int s = 0; s < S; ++s) sel[(size_t)r * S + s] = x[(size_t)r * V + idx[(size_t)r * S + s]] - z;
    }
    return 0;
}

/* gx[r][v] = -softmax(x[r])[v] * sum_s g[r][s] + sum_{s: idx[r][s]==v} g[r][s]. */
int dagref_lsg_bwd_f64(const double *x, const int64_t *idx, const double *g, int rows, int V, int S,
                       double *gx) {
    for (int r = 0; r < rows; ++r) {
        double z = lse_pair_sum(x + (size_t)r * V, V);
        double G = 0.0;
        for (int s = 0; s < S; ++s) G += g[(size_t)r * S + s];
        for (int v = 0; v < V; ++v) gx[(size_t)r * V + v] = -exp(x[(size_t)r * V + v] - z) * G;
        for (int s = 0; s < S; ++s) gx[(size_t)r * V + idx[(size_t)r * S + s]] += g[(size_t)r * S + s];
    }
    return 0;
}

// The three operators for float64 tensors, in float64 arithmetic throughout (the reference instantiates its kernels
// for double as well: fs_plugins/custom_ops/dag_loss.cu:160, 294, 415, 499; dag_best_alignment.cu:150;
// logsoftmax_gather.cu:343-347).  Nobody trains in float64: these are the kernels a caller checks the others
// against (gradcheck, a float64 run of a small model), so they are plain -- log-domain sums with one exp per
// term, tables of absolute float64 values, one workgroup per sweep, the transitions read again from memory in every
// step (which is what bounds them) -- and share nothing with the float32 kernels.
#include <math.h>

#include "dagx_common.h"

namespace dagx {
namespace {

constexpr int kThreads = 1024;
constexpr int kTeam = 8;                       // lanes that share a node's sum
constexpr int kTeams = kThreads / kTeam;
#define DAGX_NEG_INF_D ((double)DAGX_NEG_INF)

__device__ __forceinline__ bool lengths_valid(int Lb, int Tb, int L, int T) {
    return Tb >= 1 && Lb >= 1 && Tb <= T && Lb <= L && Tb <= Lb;
}
__device__ __forceinline__ bool is_finite(double z) { return z > DAGX_NEG_INF_D && z < -DAGX_NEG_INF_D; }

// A running log-sum-exp as (maximum, sum of exp(term - maximum)).  -inf terms add nothing; a NaN term makes the
// sum a NaN for good.
__device__ __forceinline__ void lse_add(double &m, double &s, double x) {
    if (x != x) { s = x; return; }
    if (x == DAGX_NEG_INF_D) return;
    if (x > m) { s = s * exp(m - x) + 1.0; m = x; }   // (m = -inf: 0 * 0 + 1)
    else s += exp(x - m);
}
// R terms at once: their maximum first, then R independent exponentials (the one-term form above is a chain of
// dependent ones).
template <int R>
__device__ __forceinline__ void lse_add_chunk(double &m, double &s, const double (&x)[R]) {
    double cm = x[0];
    bool nan = x[0] != x[0];
#pragma unroll
    for (int r = 1; r < R; ++r) { cm = fmax(cm, x[r]); nan |= x[r] != x[r]; }
    if (nan) { s = __builtin_nan(""); return; }
    if (cm == DAGX_NEG_INF_D) return;
    const double nm = fmax(m, cm);
    double part = 0.0;
#pragma unroll
    for (int r = 0; r < R; ++r) part += exp(x[r] - nm);
    s = s * exp(m - nm) + part;   // (m = -inf: s is 0, or a NaN on its way)
    m = nm;
}
__device__ __forceinline__ void lse_merge(double &m, double &s, double mo, double so) {
    const double nm = fmax(m, mo);
    if (nm > DAGX_NEG_INF_D) s = s * exp(m - nm) + so * exp(mo - nm);
    else s += so;   // 0 + 0, or a NaN on its way
    m = nm;
}
__device__ __forceinline__ void team_lse(double &m, double &s) {   // the team's pairs into one, in every lane of the team
#pragma unroll
    for (int o = kTeam / 2; o > 0; o >>= 1) {
        const double mo = __shfl_xor(m, o, kWave), so = __shfl_xor(s, o, kWave);
        lse_merge(m, s, mo, so);
    }
}

struct LossArgs {
    const double *match; int64_t ms0, ms1, ms2;
    const double *links;
    const int64_t *out_len, *tgt_len;
    int B, T, L, translen;
    double *tab[2];   // alpha, beta: [B,T,L]; a cell holds the log-sum of the paths from the start (to the end) through it, its own match included
    double *loss;     // [B]: alpha's read-out
};

// One workgroup per (sample, direction).  Row t of a table has values on the band t <= node <= t + (L_b - T_b),
// the nodes that paths of exactly T_b nodes from 0 to L_b - 1 can occupy at step t, and -inf elsewhere; rows
// t >= T_b and the tables of samples with invalid lengths are not written.  The rows are read back from
// global memory by the workgroup that wrote them, a barrier later.
__global__ __launch_bounds__(kThreads) void loss_sweep_f64_kernel(LossArgs a) {
    const int b = blockIdx.x, dir = blockIdx.y, tid = threadIdx.x;
    const int L = a.L, translen = a.translen;
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
    if (!lengths_valid(Lb, Tb, L, a.T)) {
        if (tid == 0 && dir == 0) a.loss[b] = DAGX_NEG_INF_D;
        return;
    }
    const double *match = a.match + (int64_t)b * a.ms0;
    const double *links = a.links + (int64_t)b * L * translen;
    double *tab = a.tab[dir] + (int64_t)b * a.T * L;
    const int slack = Lb - Tb;
    const int team = tid / kTeam, sub = tid % kTeam;
    {
        const int t0 = dir ? Tb - 1 : 0, n0 = dir ? Lb - 1 : 0;
        const double m0 = match[t0 * a.ms1 + n0 * a.ms2];
        for (int n = tid; n < L; n += kThreads) tab[(int64_t)t0 * L + n] = n == n0 ? m0 : DAGX_NEG_INF_D;
    }
    __syncthreads();
    for (int s = 1; s < Tb; ++s) {
        const int t = dir ? Tb - 1 - s : s;
        const double *prev = tab + (int64_t)(dir ? t + 1 : t - 1) * L;
        double *cur = tab + (int64_t)t * L;
        for (int n = tid; n < L; n += kThreads)
            if (n < t || n > t + slack) cur[n] = DAGX_NEG_INF_D;
        for (int n = t + team; n <= t + slack; n += kTeams) {
            double m = DAGX_NEG_INF_D, sum = 0.0;
            constexpr int R = 8;   // terms in flight per lane
            double x[R];
            if (dir == 0) {   // predecessors i of node n: E[i][n] = links[i][n - i - 1]
                int lo = n - translen; if (lo < t - 1) lo = t - 1;
                for (int i0 = lo + sub; i0 < n; i0 += kTeam * R) {
#pragma unroll
                    for (int q = 0; q < R; ++q) {
                        const int i = i0 + q * kTeam, ic = i < n ? i : n - 1;   // (beyond the last predecessor: a valid address, the term dropped)
                        const double v = prev[ic] + links[(int64_t)ic * translen + (n - ic - 1)];
                        x[q] = i < n ? v : DAGX_NEG_INF_D;
                    }
                    lse_add_chunk<R>(m, sum, x);
                }
            } else {          // successors j of node n
                int hi = n + translen; if (hi > t + 1 + slack) hi = t + 1 + slack;
                const double *row = links + (int64_t)n * translen - (n + 1);
                for (int j0 = n + 1 + sub; j0 <= hi; j0 += kTeam * R) {
#pragma unroll
                    for (int q = 0; q < R; ++q) {
                        const int j = j0 + q * kTeam, jc = j <= hi ? j : hi;
                        const double v = prev[jc] + row[jc];
                        x[q] = j <= hi ? v : DAGX_NEG_INF_D;
                    }
                    lse_add_chunk<R>(m, sum, x);
                }
            }
            team_lse(m, sum);
            if (sub == 0)
                cur[n] = (m > DAGX_NEG_INF_D || sum != sum) ? (m + log(sum)) + match[t * a.ms1 + n * a.ms2] : DAGX_NEG_INF_D;
        }
        __syncthreads();
    }
    if (tid == 0 && dir == 0) a.loss[b] = tab[(int64_t)(Tb - 1) * L + (Lb - 1)];
}

struct GradArgs {
    const double *grad_out; int64_t gstride;
    const double *alpha, *beta, *loss;
    const double *match; int64_t ms0, ms1, ms2;
    const double *links;
    const int64_t *out_len, *tgt_len;
    int B, T, L, translen;
    double *grad_match, *grad_links;
};

// grad_match[b][t][j] = g_b * exp(alpha + beta - match - Z): the posterior of the cell; 0 outside the sample, where
// a table says -inf, or when Z is not finite.
__global__ __launch_bounds__(256) void grad_match_f64_kernel(GradArgs a) {
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (int64_t)a.B * a.T * a.L) return;
    const int j = (int)(id % a.L), t = (int)((id / a.L) % a.T), b = (int)(id / ((int64_t)a.L * a.T));
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
    double r = 0.0;
    if (lengths_valid(Lb, Tb, a.L, a.T) && t < Tb && j < Lb) {
        const double Z = a.loss[b], al = a.alpha[id], be = a.beta[id], m = a.match[b * a.ms0 + t * a.ms1 + j * a.ms2];
        if (is_finite(Z) && al > DAGX_NEG_INF_D && be > DAGX_NEG_INF_D && is_finite(m))
            r = a.grad_out[b * a.gstride] * exp(((al - Z) + be) - m);
    }
    a.grad_match[id] = r;
}

// grad_links[b][i][d] = g_b * sum_t exp(alpha[t][i] + E[i][d] + beta[t+1][i+d+1] - Z), every term a posterior <= 1.
// A thread per transition; the threads of a wave share alpha[t][i] and read neighbouring cells of beta.
__global__ __launch_bounds__(256) void grad_links_f64_kernel(GradArgs a) {
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (int64_t)a.B * a.L * a.translen) return;
    const int d = (int)(id % a.translen), i = (int)((id / a.translen) % a.L), b = (int)(id / ((int64_t)a.translen * a.L));
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b], j = i + d + 1;
    double r = 0.0;
    if (lengths_valid(Lb, Tb, a.L, a.T) && Tb >= 2 && j < Lb) {
        const double Z = a.loss[b], e = a.links[id];
        if (is_finite(Z) && is_finite(e)) {
            const int slack = Lb - Tb;
            int tlo = j - 1 - slack; if (tlo < 0) tlo = 0;      // beta[t+1][j] is on the band from here on
            int thi = i; if (thi > Tb - 2) thi = Tb - 2;        // alpha[t][i] is on the band up to here
            const double *al = a.alpha + (int64_t)b * a.T * a.L + i, *be = a.beta + (int64_t)b * a.T * a.L + j;
            const double k = e - Z;
            double sum = 0.0;
            for (int t = tlo; t <= thi; ++t) {
                const double x = al[(int64_t)t * a.L], y = be[(int64_t)(t + 1) * a.L];
                if (x > DAGX_NEG_INF_D && y > DAGX_NEG_INF_D) sum += exp((x + k) + y);
            }
            r = a.grad_out[b * a.gstride] * sum;
        }
    }
    a.grad_links[id] = r;
}

struct AlignArgs {
    const double *match; int64_t ms0, ms1, ms2;
    const double *links;
    const int64_t *out_len, *tgt_len;
    int B, T, L, translen;
    double *score;    // [B,T,L] workspace
    int64_t *path;    // [B,L]
};

// Viterbi, one workgroup per sample: score[t][j] = fl(max_i fl(score[t-1][i] + E[i][j]) + match[t][j]), the two
// roundings of the torch-native recurrence (fs_plugins/custom_ops/dag_loss.py:303-320) in float64; then the first
// wave walks back from (T_b - 1, L_b - 1), taking at every step the lowest predecessor that attains the maximum
// (dag_loss.py:253-257, 350).  Samples without a finite path, or with invalid lengths, get -1 everywhere.
__global__ __launch_bounds__(kThreads) void align_f64_kernel(AlignArgs a) {
    const int b = blockIdx.x, tid = threadIdx.x;
    const int L = a.L, translen = a.translen;
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
    int64_t *path = a.path + (int64_t)b * L;
    for (int n = tid; n < L; n += kThreads) path[n] = -1;
    if (!lengths_valid(Lb, Tb, L, a.T)) return;
    const double *match = a.match + (int64_t)b * a.ms0;
    const double *links = a.links + (int64_t)b * L * translen;
    double *score = a.score + (int64_t)b * a.T * L;
    const int slack = Lb - Tb;
    const int team = tid / kTeam, sub = tid % kTeam;
    {
        const double m0 = match[0];
        for (int n = tid; n < L; n += kThreads) score[n] = n == 0 ? m0 : DAGX_NEG_INF_D;
    }
    __syncthreads();
    for (int t = 1; t < Tb; ++t) {
        const double *prev = score + (int64_t)(t - 1) * L;
        double *cur = score + (int64_t)t * L;
        for (int n = tid; n < L; n += kThreads)
            if (n < t || n > t + slack) cur[n] = DAGX_NEG_INF_D;
        for (int n = t + team; n <= t + slack; n += kTeams) {
            int lo = n - translen; if (lo < t - 1) lo = t - 1;
            double best = DAGX_NEG_INF_D;
            constexpr int R = 8;   // candidates in flight per lane
            for (int i0 = lo + sub; i0 < n; i0 += kTeam * R) {
                double c[R];
#pragma unroll
                for (int q = 0; q < R; ++q) {
                    const int i = i0 + q * kTeam, ic = i < n ? i : n - 1;
                    const double v = prev[ic] + links[(int64_t)ic * translen + (n - ic - 1)];
                    c[q] = i < n ? v : DAGX_NEG_INF_D;
                }
#pragma unroll
                for (int q = 0; q < R; ++q) best = fmax(best, c[q]);
            }
#pragma unroll
            for (int o = kTeam / 2; o > 0; o >>= 1) best = fmax(best, __shfl_xor(best, o, kWave));
            if (sub == 0) cur[n] = best + match[t * a.ms1 + n * a.ms2];
        }
        __syncthreads();
    }
    if (tid >= kWave) return;
    if (!(score[(int64_t)(Tb - 1) * L + (Lb - 1)] > DAGX_NEG_INF_D)) return;   // (path was cleared by every thread's own stores or is not read here)
    int j = Lb - 1;
    for (int t = Tb - 1; t >= 1; --t) {
        if (tid == 0) path[j] = t;
        const double *prev = score + (int64_t)(t - 1) * L;
        int lo = j - translen; if (lo < t - 1) lo = t - 1;
        double best = DAGX_NEG_INF_D; int arg = 0x7fffffff;
        for (int i = lo + tid; i < j; i += kWave) {   // ascending per lane: a strict > keeps the lane's lowest
            const double c = prev[i] + links[(int64_t)i * translen + (j - i - 1)];
            if (c > best) { best = c; arg = i; }
        }
        double top = best;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) top = fmax(top, __shfl_xor(top, o, kWave));
        int pick = best == top ? arg : 0x7fffffff;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { const int other = __shfl_xor(pick, o, kWave); pick = other < pick ? other : pick; }
        if (pick == 0x7fffffff) return;   // a NaN on the path: what is written so far stays
        j = pick;
    }
    if (tid == 0) path[j] = 0;
}

struct GatherArgs {
    double *logits;   // [rows, V]
    int64_t V; int L, S;
    const int64_t *idx; int64_t is0, is1, is2;
    double *sel; int64_t ss0, ss1, ss2;          // forward: out; backward: the incoming gradient
    double *lse;      // [rows]
};

template <typename F>
__device__ __forceinline__ void block_merge(double &m, double &s, double *lds, F merge) {   // 256 threads: every thread gets the total
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { const double mo = __shfl_xor(m, o, kWave), so = __shfl_xor(s, o, kWave); merge(m, s, mo, so); }
    __syncthreads();
    if (lane == 0) { lds[2 * wave] = m; lds[2 * wave + 1] = s; }
    __syncthreads();
    m = lds[0]; s = lds[1];
    for (int w = 1; w < 4; ++w) merge(m, s, lds[2 * w], lds[2 * w + 1]);
}

// A workgroup of 256 threads per row: log-sum-exp of the row in one pass, then the gathered entries.
__global__ __launch_bounds__(256) void lsg_fwd_f64_kernel(GatherArgs a) {
    __shared__ double lds[8];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const double *x = a.logits + row * a.V;
    double m = DAGX_NEG_INF_D, s = 0.0;
    for (int64_t v = tid; v < a.V; v += 256) lse_add(m, s, x[v]);
    block_merge(m, s, lds, [](double &m1, double &s1, double m2, double s2) { lse_merge(m1, s1, m2, s2); });
    const double lse = (m > DAGX_NEG_INF_D || s != s) ? m + log(s) : DAGX_NEG_INF_D;
    if (tid == 0 && a.lse) a.lse[row] = lse;
    const int64_t bb = row / a.L, ll = row % a.L;
    for (int q = tid; q < a.S; q += 256) {
        const int64_t id = a.idx[bb * a.is0 + ll * a.is1 + q * a.is2];
        a.sel[bb * a.ss0 + ll * a.ss1 + q * a.ss2] = (id >= 0 && id < a.V) ? x[id] - lse : __builtin_nan("");
    }
}

// The gradient, written over the row: -softmax(row)[v] * sum_s g[s], then + g[s] at the gathered ids.  Entries that
// name the same id are added in ascending order of s by the thread of the first of them, so the result does not
// depend on timing.
__global__ __launch_bounds__(256) void lsg_bwd_f64_kernel(GatherArgs a) {
    __shared__ double lds[8];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    double *x = a.logits + row * a.V;
    const int64_t bb = row / a.L, ll = row % a.L;
    const int64_t *idx = a.idx + bb * a.is0 + ll * a.is1;
    const double *g = a.sel + bb * a.ss0 + ll * a.ss1;
    double total = 0.0, unused = 0.0;
    for (int q = tid; q < a.S; q += 256) total += g[q * a.ss2];
    block_merge(total, unused, lds, [](double &m1, double &s1, double m2, double s2) { m1 += m2; s1 += s2; });
    const double lse = a.lse[row];
    for (int64_t v = tid; v < a.V; v += 256) x[v] = -exp(x[v] - lse) * total;
    __syncthreads();
    for (int q = tid; q < a.S; q += 256) {
        const int64_t id = idx[q * a.is2];
        if (id < 0 || id >= a.V) continue;
        bool first = true;
        for (int p = 0; p < q && first; ++p) first = idx[p * a.is2] != id;
        if (!first) continue;
        double add = g[q * a.ss2];
        for (int p = q + 1; p < a.S; ++p)
            if (idx[p * a.is2] == id) add += g[p * a.ss2];
        x[id] += add;
    }
}

int check_dag_args(const char *who, const void *match, const int64_t *ms, const void *links, const int64_t *ol, const int64_t *tl,
                   int B, int T, int L, int translen) {
    if (B < 0 || T < 1 || L < 1 || translen < 1) { set_error("%s: bad sizes B=%d T=%d L=%d translen=%d", who, B, T, L, translen); return DAGX_ERR_ARGUMENT; }
    if (B > 0 && (!match || !ms || !links || !ol || !tl)) { set_error("%s: null pointer argument", who); return DAGX_ERR_ARGUMENT; }
    if (B > 65535) { set_error("%s: B must not exceed 65535", who); return DAGX_ERR_UNSUPPORTED; }
    if ((int64_t)B * T * L >= ((int64_t)1 << 31) * 256 || (int64_t)B * L * translen >= ((int64_t)1 << 31) * 256) {
        set_error("%s: more cells than one launch addresses", who); return DAGX_ERR_UNSUPPORTED;
    }
    return DAGX_OK;
}

}  // namespace

size_t align_f64_workspace_bytes(int B, int T, int L) { return (size_t)B * T * L * sizeof(double); }

}  // namespace dagx

using namespace dagx;

extern "C" int dagx_loss_f64_fwd(const double *match, const int64_t match_strides[3], const double *links,
                                 const int64_t *out_len, const int64_t *tgt_len, int B, int T, int L, int translen,
                                 double *alpha, double *beta, double *loss, int require_gradient, void *stream) {
    if (int rc = check_dag_args("dagx_loss_f64_fwd", match, match_strides, links, out_len, tgt_len, B, T, L, translen)) return rc;
    if (B == 0) return DAGX_OK;
    if (!alpha || !loss || (require_gradient && !beta)) { set_error("dagx_loss_f64_fwd: null output pointer"); return DAGX_ERR_ARGUMENT; }
    LossArgs a{match, match_strides[0], match_strides[1], match_strides[2], links, out_len, tgt_len, B, T, L, translen, {alpha, beta}, loss};
    hipLaunchKernelGGL(loss_sweep_f64_kernel, dim3(B, require_gradient ? 2 : 1), dim3(kThreads), 0, (hipStream_t)stream, a);
    return check_launch("dagx_loss_f64_fwd");
}

extern "C" int dagx_loss_f64_bwd(const double *grad_out, int64_t grad_out_stride, const double *alpha, const double *beta,
                                 const double *loss, const double *match, const int64_t match_strides[3], const double *links,
                                 const int64_t *out_len, const int64_t *tgt_len, int B, int T, int L, int translen,
                                 double *grad_match, double *grad_links, void *stream) {
    if (int rc = check_dag_args("dagx_loss_f64_bwd", match, match_strides, links, out_len, tgt_len, B, T, L, translen)) return rc;
    if (B == 0) return DAGX_OK;
    if (!grad_out || !alpha || !beta || !loss) { set_error("dagx_loss_f64_bwd: null pointer argument"); return DAGX_ERR_ARGUMENT; }
    GradArgs a{grad_out, grad_out_stride, alpha, beta, loss, match, match_strides[0], match_strides[1], match_strides[2], links,
               out_len, tgt_len, B, T, L, translen, grad_match, grad_links};
    if (grad_match) {
        const int64_t n = (int64_t)B * T * L;
        hipLaunchKernelGGL(grad_match_f64_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, a);
        if (int rc = check_launch("dagx_loss_f64_bwd (grad_match)")) return rc;
    }
    if (grad_links) {
        const int64_t n = (int64_t)B * L * translen;
        hipLaunchKernelGGL(grad_links_f64_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, a);
        if (int rc = check_launch("dagx_loss_f64_bwd (grad_links)")) return rc;
    }
    return DAGX_OK;
}

extern "C" int dagx_best_alignment_f64(const double *match, const int64_t match_strides[3], const double *links,
                                       const int64_t *out_len, const int64_t *tgt_len, int B, int T, int L, int translen,
                                       int64_t *path, void *workspace, size_t workspace_bytes, void *stream) {
    if (int rc = check_dag_args("dagx_best_alignment_f64", match, match_strides, links, out_len, tgt_len, B, T, L, translen)) return rc;
    if (B == 0) return DAGX_OK;
    if (!path) { set_error("dagx_best_alignment_f64: null output pointer"); return DAGX_ERR_ARGUMENT; }
    if (!workspace || workspace_bytes < align_f64_workspace_bytes(B, T, L) || (reinterpret_cast<uintptr_t>(workspace) & 7)) {
        set_error("dagx_best_alignment_f64: workspace of %zu bytes, 8-byte aligned, required", align_f64_workspace_bytes(B, T, L));
        return DAGX_ERR_WORKSPACE;
    }
    AlignArgs a{match, match_strides[0], match_strides[1], match_strides[2], links, out_len, tgt_len, B, T, L, translen,
                static_cast<double *>(workspace), path};
    hipLaunchKernelGGL(align_f64_kernel, dim3(B), dim3(kThreads), 0, (hipStream_t)stream, a);
    return check_launch("dagx_best_alignment_f64");
}

static int check_gather_args(const char *who, const void *logits, int B, int L, int64_t V, int S, const int64_t *idx, const int64_t *is,
                             const void *sel, const int64_t *ss) {
    if (B < 0 || L < 0 || V < 1 || S < 0) { set_error("%s: bad sizes B=%d L=%d V=%lld S=%d", who, B, L, (long long)V, S); return DAGX_ERR_ARGUMENT; }
    if ((int64_t)B * L >= ((int64_t)1 << 31)) { set_error("%s: more rows than one launch addresses", who); return DAGX_ERR_UNSUPPORTED; }
    if ((int64_t)B * L > 0 && (!logits || (S > 0 && (!idx || !is || !sel || !ss)))) { set_error("%s: null pointer argument", who); return DAGX_ERR_ARGUMENT; }
    return DAGX_OK;
}

extern "C" int dagx_lsg_f64_fwd(const double *logits, int B, int L, int64_t V, int S, const int64_t *idx, const int64_t idx_strides[3],
                                double *sel, const int64_t sel_strides[3], double *lse, void *stream) {
    if (int rc = check_gather_args("dagx_lsg_f64_fwd", logits, B, L, V, S, idx, idx_strides, sel, sel_strides)) return rc;
    if ((int64_t)B * L == 0) return DAGX_OK;
    GatherArgs a{const_cast<double *>(logits), V, L, S, idx, S ? idx_strides[0] : 0, S ? idx_strides[1] : 0, S ? idx_strides[2] : 0,
                 sel, S ? sel_strides[0] : 0, S ? sel_strides[1] : 0, S ? sel_strides[2] : 0, lse};
    hipLaunchKernelGGL(lsg_fwd_f64_kernel, dim3((unsigned)((int64_t)B * L)), dim3(256), 0, (hipStream_t)stream, a);
    return check_launch("dagx_lsg_f64_fwd");
}

extern "C" int dagx_lsg_f64_bwd(double *logits_inout, int B, int L, int64_t V, int S, const int64_t *idx, const int64_t idx_strides[3],
                                const double *grad_sel, const int64_t gsel_strides[3], const double *lse, void *stream) {
    if (int rc = check_gather_args("dagx_lsg_f64_bwd", logits_inout, B, L, V, S, idx, idx_strides, grad_sel, gsel_strides)) return rc;
    if ((int64_t)B * L == 0) return DAGX_OK;
    if (!lse) { set_error("dagx_lsg_f64_bwd: lse (written by dagx_lsg_f64_fwd) is required"); return DAGX_ERR_ARGUMENT; }
    GatherArgs a{logits_inout, V, L, S, idx, S ? idx_strides[0] : 0, S ? idx_strides[1] : 0, S ? idx_strides[2] : 0,
                 const_cast<double *>(grad_sel), S ? gsel_strides[0] : 0, S ? gsel_strides[1] : 0, S ? gsel_strides[2] : 0, const_cast<double *>(lse)};
    hipLaunchKernelGGL(lsg_bwd_f64_kernel, dim3((unsigned)((int64_t)B * L)), dim3(256), 0, (hipStream_t)stream, a);
    return check_launch("dagx_lsg_f64_bwd");
}

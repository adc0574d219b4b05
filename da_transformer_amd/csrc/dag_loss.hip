// DAG loss on gfx950: log-semiring alpha/beta sweeps and the two gradient kernels.
//
//   alpha[t][j] = LSE_{i<j, j-i<=translen}(alpha[t-1][i] + E[i][j]) + match[t][j],  alpha[0][0] = match[0][0]
//   beta [t][i] = LSE_{j>i, j-i<=translen}(E[i][j] + beta[t+1][j]) + match[t][i],   beta[T_b-1][L_b-1] = match[..]
//   E[i][j] = links[i][j-i-1] ("shifted" layout), accumulation in fp32 whatever the input dtype.
//
// Sweeps ("exact" path): one workgroup per (sample, direction); the T-1 dependent steps are
// separated by workgroup barriers only, the running vector lives in LDS, every term is evaluated
// in the log domain (max pass + exp-sum pass over register-resident chunks).  Only the band of
// cells that can lie on a complete path, t <= j <= L_b - T_b + t, is evaluated; everything else
// is written as -inf.
#include "dagx_common.h"

namespace dagx {

struct SweepArgs {
    const void *match; int64_t ms0, ms1, ms2;
    const void *links;
    const int64_t *out_len, *tgt_len;
    int B, T, L, translen;
    float *alpha, *beta, *loss;
};

__device__ __forceinline__ bool lengths_ok(int Lb, int Tb, int L, int T) {
    return Tb >= 1 && Lb >= 1 && Tb <= T && Lb <= L && Tb <= Lb;
}

// Chunk of R predecessor terms held in registers: max pass, then exp-sum pass; merged into (m,s).
template <int R>
__device__ __forceinline__ void lse_chunk(const float (&x)[R], float &m, float &s) {
    float cm = x[0];
#pragma unroll
    for (int r = 1; r < R; ++r) cm = fmaxf(cm, x[r]);
    if (cm == DAGX_NEG_INF) return;
    float nm = fmaxf(m, cm);
    float part = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) part += fast_exp2((x[r] - nm) * kLog2e);
    s = s * fast_exp2((m - nm) * kLog2e) + part;  // m = -inf gives 0 * 0
    m = nm;
}

template <typename TM, typename TL, int NT>
__global__ __launch_bounds__(NT) void dag_sweep_kernel(SweepArgs a) {
    extern __shared__ float lds_f[];  // two vectors of L floats
    const int b = blockIdx.x;
    const int dir = blockIdx.y;  // 0: alpha, 1: beta
    const int tid = threadIdx.x;
    const int L = a.L, T = a.T, translen = a.translen;
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
    const TM *match = static_cast<const TM *>(a.match) + (int64_t)b * a.ms0;
    const TL *links = static_cast<const TL *>(a.links) + (int64_t)b * L * translen;
    float *out = (dir == 0 ? a.alpha : a.beta) + (int64_t)b * T * L;
    float *fprev = lds_f, *fcur = lds_f + L;

    if (!lengths_ok(Lb, Tb, L, T)) {
        for (int64_t k = tid; k < (int64_t)T * L; k += NT) out[k] = DAGX_NEG_INF;
        if (dir == 0 && tid == 0) a.loss[b] = DAGX_NEG_INF;
        return;
    }
    const int slack = Lb - Tb;  // band: t <= j <= slack + t

    if (dir == 0) {
        // ---------------- alpha: thread <-> column j, loop over predecessors i ----------------
        const float first = to_float(match[0]);
        for (int j = tid; j < L; j += NT) {
            float v = (j == 0) ? first : DAGX_NEG_INF;
            fprev[j] = v;
            out[j] = v;
        }
        __syncthreads();
        for (int t = 1; t < Tb; ++t) {
            const int jhi = slack + t;
            for (int j = tid; j < L; j += NT) {
                float val = DAGX_NEG_INF;
                if (j >= t && j <= jhi) {
                    int ilo = j - translen; if (ilo < t - 1) ilo = t - 1;
                    float m = DAGX_NEG_INF, s = 0.f;
                    constexpr int R = 16;
                    // address of E[i][j-i-1] = links + i*(translen-1) + (j-1)
                    const TL *col = links + (j - 1);
                    const int64_t rs = translen - 1;
                    for (int i0 = ilo; i0 < j; i0 += R) {
                        float x[R];
#pragma unroll
                        for (int r = 0; r < R; ++r) {
                            int i = i0 + r;
                            int ic = i < j ? i : j - 1;
                            float e = to_float(col[(int64_t)ic * rs]);
                            x[r] = i < j ? fprev[ic] + e : DAGX_NEG_INF;
                        }
                        lse_chunk<R>(x, m, s);
                    }
                    if (m > DAGX_NEG_INF)
                        val = (m + fast_log2(s) * kLn2) + to_float(match[(int64_t)t * a.ms1 + (int64_t)j * a.ms2]);
                }
                fcur[j] = val;
                out[(int64_t)t * L + j] = val;
            }
            __syncthreads();
            float *sw = fprev; fprev = fcur; fcur = sw;
        }
        if (tid == 0) a.loss[b] = fprev[Lb - 1];
        for (int64_t k = (int64_t)Tb * L + tid; k < (int64_t)T * L; k += NT) out[k] = DAGX_NEG_INF;
    } else {
        // ---------------- beta: wave <-> row i, lanes over successors j -----------------------
        const int lane = tid & (kWave - 1), wave = tid / kWave;
        constexpr int NW = NT / kWave;
        const float last = to_float(match[(int64_t)(Tb - 1) * a.ms1 + (int64_t)(Lb - 1) * a.ms2]);
        for (int j = tid; j < L; j += NT) {
            float v = (j == Lb - 1) ? last : DAGX_NEG_INF;
            fprev[j] = v;
            out[(int64_t)(Tb - 1) * L + j] = v;
        }
        for (int64_t k = (int64_t)Tb * L + tid; k < (int64_t)T * L; k += NT) out[k] = DAGX_NEG_INF;
        __syncthreads();
        for (int t = Tb - 2; t >= 0; --t) {
            const int jtop = slack + t + 1;  // successors live in the band of step t+1
            for (int i = wave; i < L; i += NW) {
                float val = DAGX_NEG_INF;
                if (i >= t && i <= slack + t) {
                    int jmax = i + translen; if (jmax > jtop) jmax = jtop;
                    const TL *row = links + (int64_t)i * translen;
                    float m = DAGX_NEG_INF, s = 0.f;
                    constexpr int R = 4;
                    for (int j0 = i + 1 + lane; j0 <= jmax; j0 += kWave * R) {  // per-lane trip counts differ by at most one
                        float x[R];
#pragma unroll
                        for (int r = 0; r < R; ++r) {
                            int j = j0 + r * kWave;
                            int jc = j <= jmax ? j : j0;
                            float e = to_float(row[jc - i - 1]);
                            x[r] = j <= jmax ? fprev[jc] + e : DAGX_NEG_INF;
                        }
                        lse_chunk<R>(x, m, s);
                    }
                    float wm = wave_max(m);
                    if (wm > DAGX_NEG_INF) {
                        float ws = wave_sum(s * fast_exp2((m - wm) * kLog2e));
                        val = (wm + fast_log2(ws) * kLn2) + to_float(match[(int64_t)t * a.ms1 + (int64_t)i * a.ms2]);
                    }
                }
                if (lane == 0) {
                    fcur[i] = val;
                    out[(int64_t)t * L + i] = val;
                }
            }
            __syncthreads();
            float *sw = fprev; fprev = fcur; fcur = sw;
        }
    }
}

// grad_match[b][t][j] = g_b * exp(alpha + beta - match - Z), Z = beta[b][0][0]; 0 outside the sample,
// where match is +-inf, or when Z is not finite.
template <typename TM>
__global__ __launch_bounds__(256) void dag_grad_match_kernel(
    const float *__restrict__ grad_out, int64_t gstride, const float *__restrict__ alpha,
    const float *__restrict__ beta, const TM *__restrict__ match, int64_t ms0, int64_t ms1, int64_t ms2,
    const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len, int T, int L,
    TM *__restrict__ grad_match) {
    const int b = blockIdx.z, t = blockIdx.y;
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= L) return;
    const int Lb = (int)out_len[b], Tb = (int)tgt_len[b];
    const int64_t o = ((int64_t)b * T + t) * L + j;
    float r = 0.f;
    if (lengths_ok(Lb, Tb, L, T) && t < Tb && j < Lb) {
        const float Z = beta[(int64_t)b * T * L];
        const float m = to_float(match[b * ms0 + t * ms1 + j * ms2]);
        if (Z > DAGX_NEG_INF && Z < __builtin_huge_valf() && m > DAGX_NEG_INF && m < __builtin_huge_valf()) {
            float x = ((alpha[o] - Z) + beta[o]) - m;
            r = grad_out[b * gstride] * fast_exp2(x * kLog2e);
        }
    }
    grad_match[o] = from_float<TM>(r);
}

// grad_links[b][i][d] = g_b * sum_{t=0}^{T_b-2} exp(alpha[t][i] + E[i][d] + beta[t+1][i+d+1] - Z).
// Tile: RI rows x 64 transitions per workgroup; the alpha columns and beta band it needs are
// staged in LDS once and every output is a T-deep exp-sum in the direct form (each term <= 1).
template <typename TL, int RI>
__global__ __launch_bounds__(256) void dag_grad_links_kernel(
    const float *__restrict__ grad_out, int64_t gstride, const float *__restrict__ alpha,
    const float *__restrict__ beta, const TL *__restrict__ links,
    const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len, int T, int L, int translen,
    TL *__restrict__ grad_links) {
    extern __shared__ float lds_g[];
    constexpr int JW = 64 + RI;          // columns of beta touched by the tile (j = i+d+1)
    float *a_s = lds_g;                  // [T][RI]
    float *b_s = lds_g + (size_t)T * RI; // [T][JW]  (row t holds beta[t][...]; row 0 unused)
    const int b = blockIdx.z;
    const int i0 = blockIdx.y * RI, d0 = blockIdx.x * 64;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int Lb = (int)out_len[b], Tb = (int)tgt_len[b];
    TL *gl = grad_links + (int64_t)b * L * translen;
    const int d = d0 + lane;
    const bool ok = lengths_ok(Lb, Tb, L, T);
    const float Z = ok ? beta[(int64_t)b * T * L] : DAGX_NEG_INF;
    const bool live = ok && Z > DAGX_NEG_INF && Z < __builtin_huge_valf() && i0 < Lb - 1 && i0 + d0 + 1 < Lb && Tb >= 2;
    if (!live) {  // whole tile is zero
        for (int r = w; r < RI; r += 4) {
            int i = i0 + r;
            if (i < L && d < translen) gl[(int64_t)i * translen + d] = from_float<TL>(0.f);
        }
        return;
    }
    const int slack = Lb - Tb;
    const int jbase = i0 + d0 + 1;
    // useful steps for this tile: t in [tlo, thi]
    int tlo = jbase - 1 - slack; if (tlo < 0) tlo = 0;
    int thi = i0 + RI - 1; if (thi > Tb - 2) thi = Tb - 2;
    const float *al = alpha + (int64_t)b * T * L, *be = beta + (int64_t)b * T * L;
    for (int k = tid; k < (thi - tlo + 1) * RI; k += 256) {
        int t = tlo + k / RI, r = k % RI;
        int i = i0 + r;
        a_s[t * RI + r] = i < Lb ? al[(int64_t)t * L + i] - Z : DAGX_NEG_INF;
    }
    for (int k = tid; k < (thi - tlo + 1) * JW; k += 256) {
        int t = tlo + 1 + k / JW, c = k % JW;
        int j = jbase + c;
        b_s[t * JW + c] = j < Lb ? be[(int64_t)t * L + j] : DAGX_NEG_INF;
    }
    __syncthreads();
    const float g = grad_out[b * gstride];
    for (int r = w; r < RI; r += 4) {
        const int i = i0 + r;
        if (i >= L || d >= translen) continue;
        const int j = i + d + 1;
        float acc = 0.f;
        if (i < Lb - 1 && j < Lb) {
            const float e = to_float(links[((int64_t)b * L + i) * translen + d]);
            if (e > DAGX_NEG_INF) {
                int t1 = i < thi ? i : thi;  // alpha[t][i] is -inf for t > i
                const int c = r + lane;      // j - jbase
                for (int t = tlo; t <= t1; ++t) {
                    float x = (a_s[t * RI + r] + b_s[(t + 1) * JW + c]) + e;
                    acc += fast_exp2(x * kLog2e);
                }
            }
        }
        gl[(int64_t)i * translen + d] = from_float<TL>(g * acc);
    }
}

// ---- host side ------------------------------------------------------------------------------
static int check_common(const void *match, int mdt, const int64_t *ms, const void *links, int ldt,
                        const int64_t *ol, const int64_t *tl, int B, int T, int L, int translen, const char *who) {
    if (!match || !ms || !links || !ol || !tl) { set_error("%s: null pointer argument", who); return DAGX_ERR_ARGUMENT; }
    if (B < 0 || T < 1 || L < 1 || translen < 1) { set_error("%s: bad sizes B=%d T=%d L=%d translen=%d", who, B, T, L, translen); return DAGX_ERR_ARGUMENT; }
    if (mdt < DAGX_F32 || mdt > DAGX_BF16 || ldt < DAGX_F32 || ldt > DAGX_BF16) { set_error("%s: unsupported dtype", who); return DAGX_ERR_ARGUMENT; }
    if (L > 8192) { set_error("%s: graph size L=%d exceeds the supported 8192", who, L); return DAGX_ERR_UNSUPPORTED; }
    if (B > 65535 || T > 65535) { set_error("%s: B and T must not exceed 65535", who); return DAGX_ERR_UNSUPPORTED; }
    return DAGX_OK;
}

template <typename TM, typename TL>
static int launch_sweeps(const SweepArgs &a, bool with_beta, hipStream_t st) {
    constexpr int NT = 1024;
    size_t lds = (size_t)a.L * 2 * sizeof(float);
    hipLaunchKernelGGL((dag_sweep_kernel<TM, TL, NT>), dim3(a.B, with_beta ? 2 : 1), dim3(NT), lds, st, a);
    return check_launch("dag_sweep");
}

template <typename TM>
static int dispatch_links(int ldt, const SweepArgs &a, bool with_beta, hipStream_t st) {
    switch (ldt) {
        case DAGX_F32: return launch_sweeps<TM, float>(a, with_beta, st);
        case DAGX_F16: return launch_sweeps<TM, __half>(a, with_beta, st);
        default: return launch_sweeps<TM, bf16_t>(a, with_beta, st);
    }
}

template <typename TM>
static int launch_grad_match(const float *go, int64_t gs, const float *al, const float *be, const void *match,
                             const int64_t *ms, const int64_t *ol, const int64_t *tl, int B, int T, int L,
                             void *gm, hipStream_t st) {
    hipLaunchKernelGGL((dag_grad_match_kernel<TM>), dim3((L + 255) / 256, T, B), dim3(256), 0, st, go, gs, al, be,
                       static_cast<const TM *>(match), ms[0], ms[1], ms[2], ol, tl, T, L, static_cast<TM *>(gm));
    return check_launch("dag_grad_match");
}

template <typename TL>
static int launch_grad_links(const float *go, int64_t gs, const float *al, const float *be, const void *links,
                             const int64_t *ol, const int64_t *tl, int B, int T, int L, int translen,
                             void *gl, hipStream_t st) {
    constexpr int RI = 32;
    size_t lds = ((size_t)T * RI + (size_t)(T + 1) * (64 + RI)) * sizeof(float);
    if (lds > 150 * 1024) { set_error("dag_loss_bwd: T=%d too large for the gradient tile", T); return DAGX_ERR_UNSUPPORTED; }
    auto kern = dag_grad_links_kernel<TL, RI>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) { set_error("dag_loss_bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); return DAGX_ERR_LAUNCH; }
    }
    hipLaunchKernelGGL(kern, dim3((translen + 63) / 64, (L + RI - 1) / RI, B), dim3(256), lds, st, go, gs, al, be,
                       static_cast<const TL *>(links), ol, tl, T, L, translen, static_cast<TL *>(gl));
    return check_launch("dag_grad_links");
}

}  // namespace dagx

using namespace dagx;

extern "C" int dagx_loss_fwd(const void *match, int match_dtype, const int64_t match_strides[3],
                             const void *links, int links_dtype,
                             const int64_t *out_len, const int64_t *tgt_len,
                             int B, int T, int L, int translen,
                             float *alpha, float *beta, float *loss,
                             void *workspace, size_t workspace_bytes, void *stream) {
    (void)workspace; (void)workspace_bytes;
    int rc = check_common(match, match_dtype, match_strides, links, links_dtype, out_len, tgt_len, B, T, L, translen, "dag_loss_fwd");
    if (rc) return rc;
    if (!alpha || !loss) { set_error("dag_loss_fwd: alpha and loss must be given"); return DAGX_ERR_ARGUMENT; }
    if (B == 0) return DAGX_OK;
    SweepArgs a{match, match_strides[0], match_strides[1], match_strides[2], links, out_len, tgt_len,
                B, T, L, translen, alpha, beta, loss};
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (match_dtype) {
        case DAGX_F32: return dispatch_links<float>(links_dtype, a, beta != nullptr, st);
        case DAGX_F16: return dispatch_links<__half>(links_dtype, a, beta != nullptr, st);
        default: return dispatch_links<bf16_t>(links_dtype, a, beta != nullptr, st);
    }
}

extern "C" int dagx_loss_bwd(const float *grad_out, int64_t grad_out_stride,
                             const float *alpha, const float *beta,
                             const void *match, int match_dtype, const int64_t match_strides[3],
                             const void *links, int links_dtype,
                             const int64_t *out_len, const int64_t *tgt_len,
                             int B, int T, int L, int translen,
                             void *grad_match, void *grad_links,
                             void *workspace, size_t workspace_bytes, void *stream) {
    (void)workspace; (void)workspace_bytes;
    int rc = check_common(match, match_dtype, match_strides, links, links_dtype, out_len, tgt_len, B, T, L, translen, "dag_loss_bwd");
    if (rc) return rc;
    if (!grad_out || !alpha || !beta) { set_error("dag_loss_bwd: grad_out, alpha and beta must be given"); return DAGX_ERR_ARGUMENT; }
    if (B == 0) return DAGX_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (grad_match) {
        switch (match_dtype) {
            case DAGX_F32: rc = launch_grad_match<float>(grad_out, grad_out_stride, alpha, beta, match, match_strides, out_len, tgt_len, B, T, L, grad_match, st); break;
            case DAGX_F16: rc = launch_grad_match<__half>(grad_out, grad_out_stride, alpha, beta, match, match_strides, out_len, tgt_len, B, T, L, grad_match, st); break;
            default: rc = launch_grad_match<bf16_t>(grad_out, grad_out_stride, alpha, beta, match, match_strides, out_len, tgt_len, B, T, L, grad_match, st); break;
        }
        if (rc) return rc;
    }
    if (grad_links) {
        switch (links_dtype) {
            case DAGX_F32: rc = launch_grad_links<float>(grad_out, grad_out_stride, alpha, beta, links, out_len, tgt_len, B, T, L, translen, grad_links, st); break;
            case DAGX_F16: rc = launch_grad_links<__half>(grad_out, grad_out_stride, alpha, beta, links, out_len, tgt_len, B, T, L, translen, grad_links, st); break;
            default: rc = launch_grad_links<bf16_t>(grad_out, grad_out_stride, alpha, beta, links, out_len, tgt_len, B, T, L, translen, grad_links, st); break;
        }
    }
    return rc;
}

// Best alignment on gfx950: max-semiring sweep with back-pointers and an on-GPU backtrack.
//
//   A[t][j] = max_{i<j, j-i<=translen} fl32(A[t-1][i] + E[i][j]) + match[t][j]   (two fp32 roundings)
//   back[t][j] = the smallest i attaining the max; backtrack from (T_b-1, L_b-1).
//
// One workgroup per sample: thread <-> node j scans its predecessors in ascending order and
// replaces the running best only on a strictly greater candidate, which is exactly the
// "lowest index among equal maxima" rule.  Back-pointers stay in LDS (16-bit) when T*L fits,
// otherwise they go to the caller's workspace.
#include "dagx_common.h"

namespace dagx {

struct AlignArgs {
    const void *match; int64_t ms0, ms1, ms2;
    const void *links;
    const int64_t *out_len, *tgt_len;
    int B, T, L, translen;
    int64_t *path;
    int32_t *trace_ws;  // [B][T][L] when the LDS variant is not used
};

template <typename TM, typename TL, int NT, bool TRACE_LDS>
__global__ __launch_bounds__(NT) void dag_align_kernel(AlignArgs a) {
    extern __shared__ float lds_a[];  // 2*L floats, then (TRACE_LDS) T*L uint16
    const int b = blockIdx.x, tid = threadIdx.x;
    const int L = a.L, T = a.T, translen = a.translen;
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
    const TM *match = static_cast<const TM *>(a.match) + (int64_t)b * a.ms0;
    const TL *links = static_cast<const TL *>(a.links) + (int64_t)b * L * translen;
    int64_t *path = a.path + (int64_t)b * L;
    float *fprev = lds_a, *fcur = lds_a + L;
    uint16_t *tr_lds = reinterpret_cast<uint16_t *>(lds_a + 2 * (size_t)L);
    int32_t *tr_glb = TRACE_LDS ? nullptr : a.trace_ws + (int64_t)b * T * L;

    for (int j = tid; j < L; j += NT) path[j] = -1;
    const bool ok = Tb >= 1 && Lb >= 1 && Tb <= T && Lb <= L && Tb <= Lb;
    if (!ok) return;
    const int slack = Lb - Tb;

    const float first = to_float(match[0]);
    for (int j = tid; j < L; j += NT) fprev[j] = (j == 0) ? first : DAGX_NEG_INF;
    __syncthreads();

    for (int t = 1; t < Tb; ++t) {
        const int jhi = slack + t;
        for (int j = tid; j < L; j += NT) {
            float val = DAGX_NEG_INF;
            int arg = 0;
            if (j >= t && j <= jhi) {
                int ilo = j - translen; if (ilo < t - 1) ilo = t - 1;
                float best = DAGX_NEG_INF;
                arg = ilo;
                constexpr int R = 16;
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
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        if (x[r] > best) { best = x[r]; arg = i0 + r; }
                }
                val = best + to_float(match[(int64_t)t * a.ms1 + (int64_t)j * a.ms2]);
            }
            fcur[j] = val;
            if (TRACE_LDS) tr_lds[(size_t)t * L + j] = (uint16_t)arg;
            else tr_glb[(int64_t)t * L + j] = arg;
        }
        __syncthreads();
        float *sw = fprev; fprev = fcur; fcur = sw;
    }

    if (tid == 0 && fprev[Lb - 1] > DAGX_NEG_INF) {
        int j = Lb - 1;
        for (int t = Tb - 1; t >= 0; --t) {
            path[j] = t;
            if (t > 0) j = TRACE_LDS ? (int)tr_lds[(size_t)t * L + j] : tr_glb[(int64_t)t * L + j];
        }
    }
}

constexpr size_t kAlignLdsBudget = 144 * 1024;

static bool trace_fits_lds(int T, int L) {
    return L <= 65535 && (size_t)L * 8 + (size_t)T * L * 2 <= kAlignLdsBudget;
}

size_t align_workspace_bytes(int B, int T, int L) {
    return trace_fits_lds(T, L) ? 0 : (size_t)B * T * L * sizeof(int32_t);
}

template <typename TM, typename TL>
static int launch_align(const AlignArgs &a, hipStream_t st) {
    constexpr int NT = 1024;
    if (trace_fits_lds(a.T, a.L)) {
        size_t lds = (size_t)a.L * 8 + (size_t)a.T * a.L * 2;
        auto kern = dag_align_kernel<TM, TL, NT, true>;
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) { set_error("dag_best_alignment: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); return DAGX_ERR_LAUNCH; }
        }
        hipLaunchKernelGGL(kern, dim3(a.B), dim3(NT), lds, st, a);
    } else {
        hipLaunchKernelGGL((dag_align_kernel<TM, TL, NT, false>), dim3(a.B), dim3(NT), (size_t)a.L * 8, st, a);
    }
    return check_launch("dag_align");
}

template <typename TM>
static int dispatch_align(int ldt, const AlignArgs &a, hipStream_t st) {
    switch (ldt) {
        case DAGX_F32: return launch_align<TM, float>(a, st);
        case DAGX_F16: return launch_align<TM, __half>(a, st);
        default: return launch_align<TM, bf16_t>(a, st);
    }
}

}  // namespace dagx

using namespace dagx;

extern "C" int dagx_best_alignment(const void *match, int match_dtype, const int64_t match_strides[3],
                                   const void *links, int links_dtype,
                                   const int64_t *out_len, const int64_t *tgt_len,
                                   int B, int T, int L, int translen,
                                   int64_t *path, void *workspace, size_t workspace_bytes, void *stream) {
    if (!match || !match_strides || !links || !out_len || !tgt_len || !path) { set_error("dag_best_alignment: null pointer argument"); return DAGX_ERR_ARGUMENT; }
    if (B < 0 || T < 1 || L < 1 || translen < 1) { set_error("dag_best_alignment: bad sizes B=%d T=%d L=%d translen=%d", B, T, L, translen); return DAGX_ERR_ARGUMENT; }
    if (match_dtype < DAGX_F32 || match_dtype > DAGX_BF16 || links_dtype < DAGX_F32 || links_dtype > DAGX_BF16) { set_error("dag_best_alignment: unsupported dtype"); return DAGX_ERR_ARGUMENT; }
    if (L > 8192) { set_error("dag_best_alignment: graph size L=%d exceeds the supported 8192", L); return DAGX_ERR_UNSUPPORTED; }
    size_t need = align_workspace_bytes(B, T, L);
    if (need > 0 && (!workspace || workspace_bytes < need)) { set_error("dag_best_alignment: workspace of %zu bytes required, %zu given", need, workspace_bytes); return DAGX_ERR_WORKSPACE; }
    if (B == 0) return DAGX_OK;
    AlignArgs a{match, match_strides[0], match_strides[1], match_strides[2], links, out_len, tgt_len,
                B, T, L, translen, path, static_cast<int32_t *>(workspace)};
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (match_dtype) {
        case DAGX_F32: return dispatch_align<float>(links_dtype, a, st);
        case DAGX_F16: return dispatch_align<__half>(links_dtype, a, st);
        default: return dispatch_align<bf16_t>(links_dtype, a, st);
    }
}

extern "C" size_t dagx_workspace_bytes(int op, int B, int T, int L, int translen) {
    if (B <= 0 || T <= 0 || L <= 0) return 0;
    if (op == DAGX_OP_BEST_ALIGNMENT) return align_workspace_bytes(B, T, L);
    if (op == DAGX_OP_LOSS_FWD) return loss_fwd_workspace_bytes(B, T, L, translen);
    if (op == DAGX_OP_LOSS_BWD) return loss_bwd_workspace_bytes(B);
    return 0;
}

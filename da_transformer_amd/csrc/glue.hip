// The criterion's elementwise glue around the DAG operators, one launch each instead of a chain
// of tensor operations over [B,T,L] and [B,L]:
//   * force_emit: pinning nodes to targets by rewriting `match`
//     (fs_plugins/criterions/nat_dag_loss.py:111-120) and the gradient rule that goes with it;
//   * glancing: best path -> reference tokens, count of already right predictions, keep
//     probability, keep mask, the second pass's decoder input and force_emit
//     (fs_plugins/criterions/nat_dag_loss.py:273-278, 307-311).
// Integer and byte work, bit-exact against the tensor formulation; the one floating-point value
// (the keep probability) repeats its float32 operation order: (float(n) / float(T_b)) * float(p).
#include "dagx_common.h"

namespace dagx {

// ---------------------------------------------------------------------------------------------
// force_emit.  force_emit[b][j] = t >= 0 pins node j to target t.  A target row is "forced" when
// any node names it; forced rows become 0 at the naming nodes and -inf elsewhere, other rows pass
// through (+0.0, as the tensor formulation adds a zero tensor).  kGrad: the same row rule applied
// to a gradient -- forced rows carry none, other rows pass unchanged.
// One workgroup handles kForceRows target rows of one sample: a pass over force_emit[b][:] marks
// which of them are forced, then the rows are rewritten.
// ---------------------------------------------------------------------------------------------
constexpr int kForceRows = 8;
constexpr int kGlueThreads = 256;

template <typename TM, bool kGrad>
__global__ __launch_bounds__(kGlueThreads) void force_emit_kernel(
    const TM *__restrict__ in, int64_t s0, int64_t s1, int64_t s2,
    const int64_t *__restrict__ force_emit, int T, int L, TM *__restrict__ out) {
    __shared__ int forced[kForceRows];
    const int b = blockIdx.y, t0 = blockIdx.x * kForceRows;
    const int64_t *fe = force_emit + (int64_t)b * L;
    if (threadIdx.x < kForceRows) forced[threadIdx.x] = 0;
    __syncthreads();
    for (int j = threadIdx.x; j < L; j += kGlueThreads) {
        const int64_t t = fe[j] - t0;
        if (t >= 0 && t < kForceRows) forced[t] = 1;
    }
    __syncthreads();
    const int rows = min(kForceRows, T - t0);
    for (int r = 0; r < rows; ++r) {
        const int t = t0 + r;
        const bool f = forced[r] != 0;
        const TM *src = in + b * s0 + t * s1;
        TM *dst = out + ((int64_t)b * T + t) * L;
        for (int j = threadIdx.x; j < L; j += kGlueThreads) {
            if (kGrad) {
                dst[j] = f ? from_float<TM>(0.0f) : src[j * s2];
            } else {
                const float v = f ? (fe[j] == t ? 0.0f : DAGX_NEG_INF) : to_float(src[j * s2]) + 0.0f;
                dst[j] = from_float<TM>(v);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Glancing.  One workgroup per sample.
//   stage 1: oracle[j] = tgt[max(path[j], 0)];  same_num = #{j: path[j] >= 0, not pinned,
//            pred[j] == oracle[j]};  pinned = #{j: prev_mask[j]}
//   keep probability (when none is given): ((T_b - pinned - same_num) / T_b * p) on assigned
//            nodes, 0 elsewhere
//   stage 2: keep[j] = rand[j] < keep_prob[j] or pinned;  tokens[j] = keep ? oracle[j] : prev[j];
//            next_force_emit[j] = keep ? path[j] : -1
// ---------------------------------------------------------------------------------------------
struct GlatArgs {
    const int64_t *path, *tgt_tokens, *pred_tokens, *prev_tokens;
    const uint8_t *prev_mask;        // may be null: nothing pinned
    const int64_t *tgt_len;
    const float *rand, *keep_prob_in;
    float context_p;
    int T, L, stages;
    int64_t *oracle, *same_num;
    float *keep_prob;
    uint8_t *keep_mask;
    int64_t *glat_tokens, *next_force_emit;
};

__global__ __launch_bounds__(kGlueThreads) void glat_glance_kernel(GlatArgs a) {
    __shared__ int part[2][kGlueThreads / kWave];
    const int b = blockIdx.x;
    const int64_t row = (int64_t)b * a.L;
    const int64_t *path = a.path + row;
    int64_t *oracle = a.oracle + row;
    const uint8_t *pinned_at = a.prev_mask ? a.prev_mask + row : nullptr;
    float prob = 0.0f;
    if (a.stages & 1) {
        const int64_t *tgt = a.tgt_tokens + (int64_t)b * a.T;
        int same = 0, pinned = 0;
        for (int j = threadIdx.x; j < a.L; j += kGlueThreads) {
            const int64_t at = path[j];
            const int64_t tok = tgt[at < 0 ? 0 : (at < a.T ? at : a.T - 1)];
            const bool pin = pinned_at && pinned_at[j];
            oracle[j] = tok;
            pinned += pin;
            same += (at >= 0 && !pin && a.pred_tokens[row + j] == tok);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { same += __shfl_xor(same, o, kWave); pinned += __shfl_xor(pinned, o, kWave); }
        if ((threadIdx.x & (kWave - 1)) == 0) { part[0][threadIdx.x / kWave] = same; part[1][threadIdx.x / kWave] = pinned; }
        __syncthreads();
        same = 0; pinned = 0;
#pragma unroll
        for (int w = 0; w < kGlueThreads / kWave; ++w) { same += part[0][w]; pinned += part[1][w]; }
        if (threadIdx.x == 0) a.same_num[b] = same;
        if ((a.stages & 2) && !a.keep_prob_in) {
            const int64_t tl = a.tgt_len[b];
            prob = ((float)(tl - pinned - same) / (float)tl) * a.context_p;
        }
    }
    if (!(a.stages & 2)) return;
    for (int j = threadIdx.x; j < a.L; j += kGlueThreads) {
        const int64_t at = path[j];
        float kp;
        if (a.keep_prob_in) kp = a.keep_prob_in[row + j];
        else { kp = prob * (at >= 0 ? 1.0f : 0.0f); a.keep_prob[row + j] = kp; }
        const bool keep = (a.rand[row + j] < kp) || (pinned_at && pinned_at[j]);
        a.keep_mask[row + j] = keep;
        a.glat_tokens[row + j] = keep ? oracle[j] : a.prev_tokens[row + j];
        a.next_force_emit[row + j] = keep ? at : -1;
    }
}

template <typename TM>
static int launch_force_emit(const void *in, const int64_t *s, const int64_t *fe, int B, int T, int L, bool grad, void *out, hipStream_t st) {
    const dim3 grid((unsigned)((T + kForceRows - 1) / kForceRows), (unsigned)B), block(kGlueThreads);
    if (grad)
        hipLaunchKernelGGL((force_emit_kernel<TM, true>), grid, block, 0, st, static_cast<const TM *>(in), s[0], s[1], s[2], fe, T, L, static_cast<TM *>(out));
    else
        hipLaunchKernelGGL((force_emit_kernel<TM, false>), grid, block, 0, st, static_cast<const TM *>(in), s[0], s[1], s[2], fe, T, L, static_cast<TM *>(out));
    return check_launch("force_emit");
}

}  // namespace dagx

using namespace dagx;

extern "C" int dagx_force_emit(const void *match, int dtype, const int64_t strides[3], const int64_t *force_emit,
                               int B, int T, int L, int gradient, void *out, void *stream) {
    if (B < 0 || T < 1 || L < 1) { set_error("dag_force_emit: bad sizes B=%d T=%d L=%d", B, T, L); return DAGX_ERR_ARGUMENT; }
    if (dtype < DAGX_F32 || dtype > DAGX_BF16) { set_error("dag_force_emit: unsupported dtype"); return DAGX_ERR_ARGUMENT; }
    if (B > 65535) { set_error("dag_force_emit: batch %d exceeds the 65535 of one launch", B); return DAGX_ERR_UNSUPPORTED; }
    if (B == 0) return DAGX_OK;
    if (!match || !strides || !force_emit || !out) { set_error("dag_force_emit: null pointer argument"); return DAGX_ERR_ARGUMENT; }
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case DAGX_F32: return launch_force_emit<float>(match, strides, force_emit, B, T, L, gradient != 0, out, st);
        case DAGX_F16: return launch_force_emit<__half>(match, strides, force_emit, B, T, L, gradient != 0, out, st);
        default: return launch_force_emit<bf16_t>(match, strides, force_emit, B, T, L, gradient != 0, out, st);
    }
}

extern "C" int dagx_glat_glance(const int64_t *path, const int64_t *tgt_tokens, const int64_t *pred_tokens,
                                const int64_t *prev_output_tokens, const uint8_t *prev_mask, const int64_t *tgt_len,
                                const float *rand, const float *keep_prob_in, float context_p,
                                int B, int T, int L, int stages,
                                int64_t *oracle, int64_t *same_num, float *keep_prob, uint8_t *keep_mask,
                                int64_t *glat_tokens, int64_t *next_force_emit, void *stream) {
    if (B < 0 || T < 1 || L < 1) { set_error("dag_glat_glance: bad sizes B=%d T=%d L=%d", B, T, L); return DAGX_ERR_ARGUMENT; }
    if (stages < 1 || stages > 3) { set_error("dag_glat_glance: stages must be 1 (oracle), 2 (mix) or 3 (both)"); return DAGX_ERR_ARGUMENT; }
    if (B == 0) return DAGX_OK;
    if (!path || !oracle) { set_error("dag_glat_glance: null pointer argument"); return DAGX_ERR_ARGUMENT; }
    if ((stages & 1) && (!tgt_tokens || !pred_tokens || !same_num)) { set_error("dag_glat_glance: the oracle stage needs tgt_tokens, pred_tokens and same_num"); return DAGX_ERR_ARGUMENT; }
    if ((stages & 2) && (!prev_output_tokens || !rand || !keep_mask || !glat_tokens || !next_force_emit)) { set_error("dag_glat_glance: the mix stage needs prev_output_tokens, rand and its three outputs"); return DAGX_ERR_ARGUMENT; }
    if ((stages & 2) && !keep_prob_in && (!(stages & 1) || !keep_prob || !tgt_len)) { set_error("dag_glat_glance: without keep_prob_in both stages must run and keep_prob and tgt_len must be given"); return DAGX_ERR_ARGUMENT; }
    GlatArgs a;
    a.path = path; a.tgt_tokens = tgt_tokens; a.pred_tokens = pred_tokens; a.prev_tokens = prev_output_tokens;
    a.prev_mask = prev_mask; a.tgt_len = tgt_len; a.rand = rand; a.keep_prob_in = keep_prob_in; a.context_p = context_p;
    a.T = T; a.L = L; a.stages = stages; a.oracle = oracle; a.same_num = same_num; a.keep_prob = keep_prob;
    a.keep_mask = keep_mask; a.glat_tokens = glat_tokens; a.next_force_emit = next_force_emit;
    hipLaunchKernelGGL(glat_glance_kernel, dim3((unsigned)B), dim3(kGlueThreads), 0, static_cast<hipStream_t>(stream), a);
    return check_launch("glat_glance");
}

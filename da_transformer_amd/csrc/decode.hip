// Greedy / lookahead decoding of the graph (decode_strategy greedy and lookahead without n-gram
// blocking, fs_plugins/models/glat_decomposed_with_link.py:691-718): every node's best successor (one
// wave per node, the whole GPU), then one workgroup per sample for the walk from node 0 to the last
// node and the token collapsing.
//   next[i] = argmax_j fl32(E[i][j] + fl32(u[j] * beta))      (lookahead; greedy: argmax_j E[i][j])
// with the lowest j among equals (the first-index rule of torch.max on the host) and two separate
// roundings as the tensor expression has them -- the product and the sum must not fuse.
#include "dagx_common.h"

namespace dagx {

constexpr int kWalkThreads = 1024;
constexpr int kWalkMaxNodes = 4096;

struct WalkArgs {
    const void *links;
    const float *node_logp;
    const int64_t *node_tokens, *out_len;
    int L, translen, greedy;
    float beta;
    int64_t pad;
    int64_t *out_tokens, *out_count, *nodes;
};

// Best successor of every node: one wave per row (b, i), lanes stride over the window, four loads in
// flight per lane.  successor: int32, sample b's row at 2 b L (the first half of the sample's row of
// int64 output tokens, which the walk kernel copies to LDS before it writes any token).
constexpr int kRowWaves = 4;

template <typename TL>
__global__ __launch_bounds__(kRowWaves * kWave) void successor_kernel(WalkArgs a, int *__restrict__ successor, int64_t rows) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t r = (int64_t)blockIdx.x * kRowWaves + wave;
    if (r >= rows) return;
    const int L = a.L, translen = a.translen;
    const int b = (int)(r / L), i = (int)(r - (int64_t)b * L);
    const TL *row = static_cast<const TL *>(a.links) + r * translen;
    const float *u = a.node_logp + (int64_t)b * L;
    const int span = min(translen, L - 1 - i);          // targets i+1 .. i+span
    float best = DAGX_NEG_INF;
    int arg = 0x7fffff;
    constexpr int kInFlight = 4;
    for (int d0 = 0; d0 < span; d0 += kWave * kInFlight) {
        float e[kInFlight], w[kInFlight];
#pragma unroll
        for (int q = 0; q < kInFlight; ++q) {
            const int d = d0 + q * kWave + lane, dc = d < span ? d : span - 1;
            e[q] = to_float(row[dc]);
            w[q] = a.greedy ? 0.0f : u[i + dc + 1];
        }
#pragma unroll
        for (int q = 0; q < kInFlight; ++q) {
            const int d = d0 + q * kWave + lane;
            const float v = a.greedy ? e[q] : __fadd_rn(e[q], __fmul_rn(w[q], a.beta));
            if (d < span && v > best) { best = v; arg = i + d + 1; }
        }
    }
    const float top = wave_max(best);
    // the lowest target among the lanes that hold the maximum; a row without any finite entry points
    // to node 0, as the arg max over a row of -inf does
    const float cand = (best == top && top > DAGX_NEG_INF) ? (float)arg : 3.0e7f;
    const int j = (int)-wave_max(-cand);
    if (lane == 0) successor[(int64_t)b * 2 * L + i] = j < L ? j : 0;
}

// The walk and the token collapsing, one workgroup per sample.
__global__ __launch_bounds__(kWalkThreads) void lookahead_walk_kernel(WalkArgs a, const int *__restrict__ successor) {
    __shared__ int next[kWalkMaxNodes];
    __shared__ int walk[kWalkMaxNodes];
    __shared__ int s_count;
    const int b = blockIdx.x, tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int L = a.L;
    const int Lb = (int)a.out_len[b];
    const int64_t *tok = a.node_tokens + (int64_t)b * L;
    int64_t *out_tokens = a.out_tokens + (int64_t)b * L;
    int64_t *nodes = a.nodes + (int64_t)b * L;
    for (int i = tid; i < L; i += kWalkThreads) next[i] = successor[(int64_t)b * 2 * L + i];
    __syncthreads();
    // the walk 0 -> next[0] -> ... until the last node (at most L nodes: a walk that does not get there,
    // which the tensor formulation would follow for ever, stops after L steps)
    if (tid == 0) {
        int j = 0, n = 1;
        walk[0] = 0;
        while (j != Lb - 1 && n < L) {
            j = next[j];
            walk[n++] = j;
        }
        s_count = n;
    }
    __syncthreads();
    const int n = s_count;
    if (wave != 0) return;
    // tokens: the first always stays; a later one when it is not the pad and differs from the one before it
    int count = 0;
    for (int k0 = 0; k0 < L; k0 += kWave) {
        const int k = k0 + lane;
        const bool in = k < n;
        const int node = in ? walk[k] : 0;
        const int64_t y = in ? tok[node] : a.pad;
        const int64_t yprev = (in && k > 0) ? tok[walk[k - 1]] : a.pad;
        const bool keep = in && (k == 0 || (y != a.pad && y != yprev));
        const unsigned long long mask = __ballot(keep);
        const int pos = count + __popcll(mask & ((1ull << lane) - 1ull));
        if (keep) out_tokens[pos] = y;
        if (k < L) nodes[k] = in ? node : -1;
        count += __popcll(mask);
    }
    if (lane == 0) a.out_count[b] = count;
    for (int k = count + lane; k < L; k += kWave) out_tokens[k] = a.pad;
}

}  // namespace dagx

using namespace dagx;

extern "C" int dagx_lookahead_decode(const void *links, int links_dtype, const float *node_logp, const int64_t *node_tokens,
                                     const int64_t *out_len, int B, int L, int translen, float beta, int greedy, int64_t pad,
                                     int64_t *out_tokens, int64_t *out_count, int64_t *nodes, void *stream) {
    if (B < 0 || L < 1 || translen < 1) { set_error("dag_lookahead_decode: bad sizes B=%d L=%d translen=%d", B, L, translen); return DAGX_ERR_ARGUMENT; }
    if (B == 0) return DAGX_OK;
    if (!links || !node_logp || !node_tokens || !out_len || !out_tokens || !out_count || !nodes) { set_error("dag_lookahead_decode: null pointer argument"); return DAGX_ERR_ARGUMENT; }
    if (links_dtype < DAGX_F32 || links_dtype > DAGX_BF16) { set_error("dag_lookahead_decode: unsupported dtype"); return DAGX_ERR_ARGUMENT; }
    if (L > kWalkMaxNodes) { set_error("dag_lookahead_decode: graph size L=%d exceeds the supported %d", L, kWalkMaxNodes); return DAGX_ERR_UNSUPPORTED; }
    WalkArgs a{links, node_logp, node_tokens, out_len, L, translen, greedy, beta, pad, out_tokens, out_count, nodes};
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the successors of sample b land in the first half of out_tokens[b] (int32 in int64 slots) and are
    // copied out of there by the walk before it writes the tokens
    int *successor = reinterpret_cast<int *>(out_tokens);
    const int64_t rows = (int64_t)B * L;
    const dim3 grid((unsigned)((rows + kRowWaves - 1) / kRowWaves)), block(kRowWaves * kWave);
    switch (links_dtype) {
        case DAGX_F32: hipLaunchKernelGGL((successor_kernel<float>), grid, block, 0, st, a, successor, rows); break;
        case DAGX_F16: hipLaunchKernelGGL((successor_kernel<__half>), grid, block, 0, st, a, successor, rows); break;
        default: hipLaunchKernelGGL((successor_kernel<bf16_t>), grid, block, 0, st, a, successor, rows); break;
    }
    int rc = check_launch("lookahead_successor");
    if (rc) return rc;
    hipLaunchKernelGGL(lookahead_walk_kernel, dim3((unsigned)B), dim3(kWalkThreads), 0, st, a, successor);
    return check_launch("lookahead_decode");
}

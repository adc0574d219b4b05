// Transition log-probabilities from per-head scores (the tail of the link predictor), gfx950.
//
//   links[b][i][d] = LSE_c( content[b][i][j][c] - LSE_{j' in win(b,i)} content[b][i][j'][c] + log_gates[b][i][c] ),
//   j = i + d + 1,  win(b,i) = { j : i < j < min(valid_end[b][i], i + 1 + translen, L) },  -inf outside the window.
//
// This is what fs_plugins/models/glat_decomposed_with_link.py:380-404 computes with a masked_fill, a
// gather into the shifted layout (:319-335), a log_softmax over the transitions, an add and a
// logsumexp over the heads -- each a pass over a [B,L,translen,H] float tensor.  Here a row (b, i) is
// read once: its window is H * n contiguous floats of `content`, held in registers by one wave (no
// LDS, no barrier: the per-head reductions run on the DPP network).
// HBM-bound: the forward reads the windows and writes [B,L,translen]; the backward reads the windows
// again and writes the gradient over the whole [B,L,L,H] tensor in place (zeros outside the windows),
// as the dense batched-GEMM backward that follows it expects.
#include <type_traits>

#include "dagx_common.h"

namespace dagx {

constexpr int kLinkThreads = 256;                 // four waves, one row each
constexpr int kLinkWaves = kLinkThreads / kWave;

// ---- 64-lane reductions on the DPP network (no LDS traffic); the result is wave-uniform ------------
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_take(float v) {   // lanes outside ROW_MASK get 0
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float lanes_sum(float v) {
    v += dpp_take<0xB1, 0xf>(v);    // quad_perm [1,0,3,2]
    v += dpp_take<0x4E, 0xf>(v);    // quad_perm [2,3,0,1]
    v += dpp_take<0x141, 0xf>(v);   // row_half_mirror
    v += dpp_take<0x140, 0xf>(v);   // row_mirror: every lane holds the sum of its row of 16
    v += dpp_take<0x142, 0xa>(v);   // row_bcast:15 into rows 1 and 3
    v += dpp_take<0x143, 0xc>(v);   // row_bcast:31 into rows 2 and 3: lane 63 holds the total
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float lanes_max(float v) {
    // (-inf is the neutral element here, so lanes a step does not reach must not contribute 0)
    auto step = [&](float t, float keep) { return fmaxf(keep, t); };
    v = step(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false)), v);
    v = step(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false)), v);
    v = step(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false)), v);
    v = step(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false)), v);
    v = step(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false)), v);
    v = step(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false)), v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// The same for H values at once, step by step across the heads: the independent chains fill each
// other's DPP wait states.
template <int H>
__device__ __forceinline__ void lanes_sum_all(float (&v)[H]) {
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] += dpp_take<0xB1, 0xf>(v[c]);
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] += dpp_take<0x4E, 0xf>(v[c]);
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] += dpp_take<0x141, 0xf>(v[c]);
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] += dpp_take<0x140, 0xf>(v[c]);
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] += dpp_take<0x142, 0xa>(v[c]);
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] += dpp_take<0x143, 0xc>(v[c]);
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v[c]), 63));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_keep(float v) {   // lanes outside ROW_MASK keep their own value
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}
template <int H>
__device__ __forceinline__ void lanes_max_all(float (&v)[H]) {
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] = fmaxf(v[c], dpp_keep<0xB1, 0xf>(v[c]));
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] = fmaxf(v[c], dpp_keep<0x4E, 0xf>(v[c]));
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] = fmaxf(v[c], dpp_keep<0x141, 0xf>(v[c]));
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] = fmaxf(v[c], dpp_keep<0x140, 0xf>(v[c]));
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] = fmaxf(v[c], dpp_keep<0x142, 0xa>(v[c]));
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] = fmaxf(v[c], dpp_keep<0x143, 0xc>(v[c]));
#pragma unroll
    for (int c = 0; c < H; ++c) v[c] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v[c]), 63));
}

// The H scores of one window position, as floats (one or two 16-byte loads for the usual H).
template <typename TC, int H>
__device__ __forceinline__ void load_heads(const TC *p, float (&x)[H]) {
    struct alignas(sizeof(TC) * H >= 16 ? 16 : sizeof(TC) * H) Pack { TC v[H]; };
    const Pack raw = *reinterpret_cast<const Pack *>(p);
#pragma unroll
    for (int c = 0; c < H; ++c) x[c] = to_float(raw.v[c]);
}
template <typename TC, int H>
__device__ __forceinline__ void store_heads(TC *p, const float (&x)[H]) {
    struct alignas(sizeof(TC) * H >= 16 ? 16 : sizeof(TC) * H) Pack { TC v[H]; };
    Pack raw;
#pragma unroll
    for (int c = 0; c < H; ++c) raw.v[c] = from_float<TC>(x[c]);
    *reinterpret_cast<Pack *>(p) = raw;
}

struct LinkRow { int b, i, jlo, n; };
__device__ __forceinline__ LinkRow link_row(const int64_t *valid_end, int64_t row, int L, int translen) {
    LinkRow r;
    r.b = (int)(row / L); r.i = (int)(row % L);
    r.jlo = r.i + 1;
    int64_t e = valid_end[row];
    int jhi = e < (int64_t)L ? (int)(e < 0 ? 0 : e) : L;
    if (jhi > r.jlo + translen) jhi = r.jlo + translen;
    r.n = jhi > r.jlo ? jhi - r.jlo : 0;
    return r;
}

// links and lse (the per-head log normalisers, [B][L][H], kept for the backward).  PER window
// positions per lane: L <= 64 * PER.
template <typename TC, int H, int PER>
__global__ __launch_bounds__(kLinkThreads) void links_fwd_kernel(
    const TC *__restrict__ content, const float *__restrict__ log_gates, const int64_t *__restrict__ valid_end,
    int64_t rows, int L, int translen, TC *__restrict__ links, float *__restrict__ lse_out) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kLinkWaves + threadIdx.x / kWave;
    if (row >= rows) return;
    // The window is loaded before valid_end is known (up to the end of the row, which always exists), so
    // that a wave waits for one memory round trip, not two; what lies past valid_end is masked afterwards.
    const int i = (int)(row % L);
    const int nmax = L - 1 - i < translen ? L - 1 - i : translen;
    const TC *win = content + (row * L + i + 1) * H;
    float x[PER][H];
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int d = lane + k * kWave;
        if (d < nmax) load_heads<TC, H>(win + (int64_t)d * H, x[k]);
    }
    const LinkRow r = link_row(valid_end, row, L, translen);
    TC *out = links + row * translen;
    if (r.n == 0) {   // no transition leaves this node
        for (int d = lane; d < translen; d += kWave) out[d] = from_float<TC>(DAGX_NEG_INF);
        if (lse_out && lane < H) lse_out[row * H + lane] = DAGX_NEG_INF;
        return;
    }
    // Chunk by chunk (64 positions), only the chunks that reach into the window are worked on (one
    // wave-uniform test per chunk and pass: rows near the end of a graph are short), and only the chunk
    // that holds the end of the window needs masking.
    // per head: maximum, then the sum of exp(x - max) = 2^(x * log2e - max * log2e), over the window
    float m[H], sum[H];
#pragma unroll
    for (int c = 0; c < H; ++c) { m[c] = DAGX_NEG_INF; sum[c] = 0.f; }
#pragma unroll
    for (int k = 0; k < PER; ++k)
        if (k * kWave < r.n) {
            if ((k + 1) * kWave > r.n) {   // the last chunk of the window
                const bool in = lane + k * kWave < r.n;
#pragma unroll
                for (int c = 0; c < H; ++c) x[k][c] = in ? x[k][c] : DAGX_NEG_INF;
            }
#pragma unroll
            for (int c = 0; c < H; ++c) m[c] = fmaxf(m[c], x[k][c]);
        }
    lanes_max_all<H>(m);
    float shift[H];   // -max * log2e; 0 for a head without any finite score: 2^(-inf) = 0, no NaN
#pragma unroll
    for (int c = 0; c < H; ++c) shift[c] = m[c] > DAGX_NEG_INF ? -m[c] * kLog2e : 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k)
        if (k * kWave < r.n)
#pragma unroll
            for (int c = 0; c < H; ++c) sum[c] += fast_exp2(__builtin_fmaf(x[k][c], kLog2e, shift[c]));
    lanes_sum_all<H>(sum);
    // bias = (log_gate - lse) in base 2 is what is added to a score of head c (a head without any
    // finite score drops out)
    float bias[H];
    bool any_head = false;
#pragma unroll
    for (int c = 0; c < H; ++c) {
        const float lse2 = m[c] > DAGX_NEG_INF ? fast_log2(sum[c]) - shift[c] : DAGX_NEG_INF;
        if (lse_out && lane == 0) lse_out[row * H + c] = lse2 * kLn2;
        bias[c] = lse2 > DAGX_NEG_INF ? __builtin_fmaf(log_gates[row * H + c], kLog2e, -lse2) : DAGX_NEG_INF;
        any_head = any_head || lse2 > DAGX_NEG_INF;
    }
    // mix the heads: log2 sum_c 2^(x * log2e + bias_c), lane-local.  Every term is at most 1 (a score
    // never exceeds its head's normaliser, a gate log-probability is at most 0), so no maximum is needed
    // unless all terms underflow -- a transition less likely than 2^-126 -- which takes the exact route.
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int d = lane + k * kWave;
        if (k * kWave >= translen) break;
        float v = DAGX_NEG_INF;
        if (k * kWave < r.n) {
            float y[H], acc = 0.f;
#pragma unroll
            for (int c = 0; c < H; ++c) { y[c] = __builtin_fmaf(x[k][c], kLog2e, bias[c]); acc += fast_exp2(y[c]); }
            if (d < r.n) {
                if (__builtin_expect(acc >= 1.17549435e-38f, 1)) v = fast_log2(acc) * kLn2;
                else if (any_head) {
                    float ym = DAGX_NEG_INF;
#pragma unroll
                    for (int c = 0; c < H; ++c) ym = fmaxf(ym, y[c]);
                    if (ym > DAGX_NEG_INF) {
                        float acc2 = 0.f;
#pragma unroll
                        for (int c = 0; c < H; ++c) acc2 += fast_exp2(y[c] - ym);
                        v = (ym + fast_log2(acc2)) * kLn2;
                    }
                }
            }
        }
        if (d < translen) out[d] = from_float<TC>(v);
    }
}

// In place: content[b][i][j][c] <- d loss / d content, 0 outside the window; grad_gates[b][i][c] =
// d loss / d log_gates.  With y = x - lse_c + g_c and w = grad_links[d] * exp(y - log sum_c' exp(y_c')):
//   d/dg_c = W_c = sum_d w[d][c],      d/dx[d][c] = w[d][c] - W_c * exp(x[d][c] - lse_c).
// The normaliser over the heads is formed again from the scores, in float32, and not taken from the stored
// `links` (which the kernel does not read): rounded to bfloat16 a link value of -6 is 0.03 off, and every weight
// of its position with it by 3 %.
template <typename TC, int H, int PER>
__global__ __launch_bounds__(kLinkThreads) void links_bwd_kernel(
    TC *__restrict__ content, const float *__restrict__ log_gates, const int64_t *__restrict__ valid_end,
    int64_t rows, int L, int translen, const TC *__restrict__ links, const float *__restrict__ lse_in,
    const TC *__restrict__ grad_links, float *__restrict__ grad_gates) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kLinkWaves + threadIdx.x / kWave;
    if (row >= rows) return;
    const LinkRow r = link_row(valid_end, row, L, translen);
    TC *full = content + row * L * H;
    float zeros[H];
#pragma unroll
    for (int c = 0; c < H; ++c) zeros[c] = 0.f;
    // outside the window: zeros (nothing of it was read)
    for (int j = lane; j < L; j += kWave)
        if (j < r.jlo || j >= r.jlo + r.n) store_heads<TC, H>(full + (int64_t)j * H, zeros);
    if (r.n == 0) {
        if (lane < H) grad_gates[row * H + lane] = 0.f;
        return;
    }
    TC *win = full + (int64_t)r.jlo * H;
    float lse[H], bias[H];
#pragma unroll
    for (int c = 0; c < H; ++c) {
        lse[c] = lse_in[row * H + c];
        bias[c] = lse[c] > DAGX_NEG_INF ? log_gates[row * H + c] - lse[c] : DAGX_NEG_INF;
    }
    // scores, incoming gradient and the link value of every window position of this lane.  When the scores of
    // a lane do not fit the register file (16 heads x 16 positions) they are not kept: the second pass reads
    // them again (from L2, the row was just read) instead of spilling them.
    constexpr bool KEEP = H * PER <= 128;
    float x[KEEP ? PER : 1][H], go[PER], lo[PER];   // lo: the link value of the position (natural log), formed in the first pass
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int d = lane + k * kWave;
        go[k] = 0.f; lo[k] = DAGX_NEG_INF;
        if (d < r.n) {
            if (KEEP) load_heads<TC, H>(win + (int64_t)d * H, x[KEEP ? k : 0]);
            go[k] = to_float(grad_links[row * translen + d]);
        } else if (KEEP) {
#pragma unroll
            for (int c = 0; c < H; ++c) x[KEEP ? k : 0][c] = DAGX_NEG_INF;
        }
    }
    auto weight = [&](const float (&xk)[H], int k, int c) -> float {   // w[d][c]
        const float y = xk[c] + bias[c];
        return (lo[k] > DAGX_NEG_INF && y > DAGX_NEG_INF) ? go[k] * fast_exp2((y - lo[k]) * kLog2e) : 0.f;
    };
    // first pass over a position: log sum_c exp(y_c) against the largest y_c (kept in lo[k]), and with the terms
    // already at hand the position's share of W_c
    auto first_pass = [&](const float (&xk)[H], int k, float (&wsum)[H]) {
        float y[H], ym = DAGX_NEG_INF;
#pragma unroll
        for (int c = 0; c < H; ++c) { y[c] = (xk[c] + bias[c]) * kLog2e; ym = fmaxf(ym, y[c]); }
        if (!(ym > DAGX_NEG_INF)) return;   // no head reaches this position (or a NaN score: the weights stay 0, as before)
        float e[H], acc = 0.f;
#pragma unroll
        for (int c = 0; c < H; ++c) { e[c] = fast_exp2(y[c] - ym); acc += e[c]; }
        lo[k] = (ym + fast_log2(acc)) * kLn2;
        const float f = go[k] / acc;
#pragma unroll
        for (int c = 0; c < H; ++c) wsum[c] += f * e[c];
    };
    float wsum[H];
#pragma unroll
    for (int c = 0; c < H; ++c) wsum[c] = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int d = lane + k * kWave;
        if (KEEP) {
            if (d < r.n) first_pass(x[KEEP ? k : 0], k, wsum);
        } else if (d < r.n) {
            float xk[H];
            load_heads<TC, H>(win + (int64_t)d * H, xk);
            first_pass(xk, k, wsum);
        }
    }
    lanes_sum_all<H>(wsum);
    if (lane < H) {
        float gsel = 0.f;
#pragma unroll
        for (int c = 0; c < H; ++c) gsel = lane == c ? wsum[c] : gsel;
        grad_gates[row * H + lane] = gsel;
    }
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int d = lane + k * kWave;
        if (d >= r.n) break;
        float xk[H], dx[H];
        if (KEEP) {
#pragma unroll
            for (int c = 0; c < H; ++c) xk[c] = x[KEEP ? k : 0][c];
        } else {
            load_heads<TC, H>(win + (int64_t)d * H, xk);
        }
#pragma unroll
        for (int c = 0; c < H; ++c) {
            const float p = (lse[c] > DAGX_NEG_INF && xk[c] > DAGX_NEG_INF) ? fast_exp2((xk[c] - lse[c]) * kLog2e) : 0.f;
            dx[c] = weight(xk, k, c) - wsum[c] * p;
        }
        store_heads<TC, H>(win + (int64_t)d * H, dx);
    }
}

static int check_links(const void *content, int dtype, const void *log_gates, const void *valid_end, int B, int L, int H,
                       int translen, const char *who) {
    if (B < 0 || L < 1 || H < 1 || translen < 1) { set_error("%s: bad sizes B=%d L=%d H=%d translen=%d", who, B, L, H, translen); return DAGX_ERR_ARGUMENT; }
    if (dtype < DAGX_F32 || dtype > DAGX_BF16) { set_error("%s: unsupported dtype", who); return DAGX_ERR_ARGUMENT; }
    if (H != 4 && H != 8 && H != 16) { set_error("%s: %d heads (4, 8 and 16 are supported)", who, H); return DAGX_ERR_UNSUPPORTED; }
    if (L > 1024) { set_error("%s: graph size L=%d exceeds the supported 1024", who, L); return DAGX_ERR_UNSUPPORTED; }
    if ((int64_t)B * L > 0x7fffffffLL) { set_error("%s: B*L too large for one launch", who); return DAGX_ERR_UNSUPPORTED; }
    if (B > 0 && (!content || !log_gates || !valid_end)) { set_error("%s: null pointer argument", who); return DAGX_ERR_ARGUMENT; }
    return DAGX_OK;
}

// window positions per lane: the smallest of 4, 8, 16 that covers the row
template <typename TC, int H>
static int launch_links_fwd(const void *content, const float *log_gates, const int64_t *valid_end, int B, int L, int translen,
                            void *links, float *lse, hipStream_t st) {
    const int64_t rows = (int64_t)B * L;
    const dim3 grid((unsigned)((rows + kLinkWaves - 1) / kLinkWaves)), block(kLinkThreads);
#define DAGX_GO(PER) hipLaunchKernelGGL((links_fwd_kernel<TC, H, PER>), grid, block, 0, st, static_cast<const TC *>(content), \
                                        log_gates, valid_end, rows, L, translen, static_cast<TC *>(links), lse)
    if (L <= 4 * kWave) DAGX_GO(4); else if (L <= 8 * kWave) DAGX_GO(8); else DAGX_GO(16);
#undef DAGX_GO
    return check_launch("links_fwd");
}
template <typename TC, int H>
static int launch_links_bwd(void *content, const float *log_gates, const int64_t *valid_end, int B, int L, int translen,
                            const void *links, const float *lse, const void *grad_links, float *grad_gates, hipStream_t st) {
    const int64_t rows = (int64_t)B * L;
    const dim3 grid((unsigned)((rows + kLinkWaves - 1) / kLinkWaves)), block(kLinkThreads);
#define DAGX_GO(PER) hipLaunchKernelGGL((links_bwd_kernel<TC, H, PER>), grid, block, 0, st, static_cast<TC *>(content), log_gates, \
                                        valid_end, rows, L, translen, static_cast<const TC *>(links), lse,                         \
                                        static_cast<const TC *>(grad_links), grad_gates)
    if (L <= 4 * kWave) DAGX_GO(4); else if (L <= 8 * kWave) DAGX_GO(8); else DAGX_GO(16);
#undef DAGX_GO
    return check_launch("links_bwd");
}

}  // namespace dagx

using namespace dagx;

#define DAGX_LINKS_DISPATCH(CALL)                                                                      \
    switch (dtype) {                                                                                   \
        case DAGX_F32: return H == 4 ? CALL(float, 4) : H == 8 ? CALL(float, 8) : CALL(float, 16);     \
        case DAGX_F16: return H == 4 ? CALL(__half, 4) : H == 8 ? CALL(__half, 8) : CALL(__half, 16);  \
        default: return H == 4 ? CALL(bf16_t, 4) : H == 8 ? CALL(bf16_t, 8) : CALL(bf16_t, 16);        \
    }

extern "C" int dagx_links_fwd(const void *content, int dtype, const float *log_gates, const int64_t *valid_end,
                              int B, int L, int H, int translen, void *links, float *lse, void *stream) {
    int rc = check_links(content, dtype, log_gates, valid_end, B, L, H, translen, "dag_links_fwd");
    if (rc) return rc;
    if (B == 0) return DAGX_OK;
    if (!links) { set_error("dag_links_fwd: the output pointer is null"); return DAGX_ERR_ARGUMENT; }
    hipStream_t st = static_cast<hipStream_t>(stream);
#define CALL(T, HH) launch_links_fwd<T, HH>(content, log_gates, valid_end, B, L, translen, links, lse, st)
    DAGX_LINKS_DISPATCH(CALL)
#undef CALL
}

extern "C" int dagx_links_bwd(void *content_inout, int dtype, const float *log_gates, const int64_t *valid_end,
                              int B, int L, int H, int translen, const void *links, const float *lse,
                              const void *grad_links, float *grad_gates, void *stream) {
    int rc = check_links(content_inout, dtype, log_gates, valid_end, B, L, H, translen, "dag_links_bwd");
    if (rc) return rc;
    if (B == 0) return DAGX_OK;
    if (!lse || !grad_links || !grad_gates) { set_error("dag_links_bwd: a saved-state or output pointer is null"); return DAGX_ERR_ARGUMENT; }
    hipStream_t st = static_cast<hipStream_t>(stream);
#define CALL(T, HH) launch_links_bwd<T, HH>(content_inout, log_gates, valid_end, B, L, translen, links, lse, grad_links, grad_gates, st)
    DAGX_LINKS_DISPATCH(CALL)
#undef CALL
}

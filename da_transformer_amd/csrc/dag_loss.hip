// DAG loss on gfx950: log-semiring alpha/beta sweeps and the two gradient kernels.
//
//   alpha[t][j] = LSE_{i<j, j-i<=translen}(alpha[t-1][i] + E[i][j]) + match[t][j],  alpha[0][0] = match[0][0]
//   beta [t][i] = LSE_{j>i, j-i<=translen}(E[i][j] + beta[t+1][j]) + match[t][i],   beta[T_b-1][L_b-1] = match[..]
//   E[i][j] = links[i][j-i-1] ("shifted" layout), accumulation in fp32 whatever the input dtype.
//
// Both sweeps run in "position space": p = node for alpha, p = L_b-1-node for beta, step s = t for
// alpha, s = T_b-1-t for beta.  In that space both are the same recurrence over predecessors
// p' < p, start at p = 0 and are read out at (s, p) = (T_b-1, L_b-1).
//
// Storage of the sweep results (what the gradient kernels consume): positions are grouped in
// blocks of 64; every (step, block) has a float64 offset and every cell a float32 residual <= 0,
//   alpha[t][node] = off[t][p/64] + hat[t][node]          (hat indexed by node, off by position block)
// so the residuals keep full fp32 resolution no matter how negative the log-likelihood is.
//
// Two sweep implementations write this format:
//   * dag_sweep_tiles_kernel ("fast"): exp(E) is staged once into registers as 64x64 tiles
//     (lane <-> output position, 64 predecessors per tile), each step is a block-scaled
//     linear-domain mat-vec done with DPP row-broadcast FMAs; the tiles of one sweep are spread
//     over a small pipeline of workgroups that hand the running vector on through global memory.
//   * dag_sweep_exact_kernel: every term evaluated in the log domain, one workgroup per sweep.
//     Handles any size and any dynamic range; it re-does the samples the fast kernel flags.
#include <atomic>
#include <cstdint>
#include <type_traits>

#include "dag_tiles.h"

namespace dagx {


struct SweepArgs {
    const void *match; int64_t ms0, ms1, ms2;
    const void *links;
    const int64_t *out_len, *tgt_len;
    int B, T, L, translen, NBK;
    float *hat[2];     // residual tables of the two sweeps of a sample (with gradients: alpha-hat, beta-hat)  [B][T][L]
    double *off[2];    // block offsets        [B][T][NBK]
    double *logz;      // [2][B] read-outs of the two sweeps (with gradients: alpha end, beta end)
    float *loss;       // [B] the read-out of sweep `loss_dir` in float
    int loss_dir;      // 0: first sweep's read-out (alpha), 1: second sweep's (beta: the partition function the backward divides by)
    int *flags;        // [B] 1 = sample must be (re)done (by the wide tile sweeps, then by the exact kernel); 2 = the wide sweeps settled it
    // fast path, all zero on entry and left zero: [0] ticket counter, [1] workgroups that have left, [2] samples the
    // float32 launch flagged (cleared by the wide launch),
    // [16 + (dir*B + b)*C + group] progress words, then [B] workgroups of the sample that have left, then [B] "risk"
    // words (a group of the sample gave up waiting for its producer)
    int *sync;
    int C;             // workgroups per sweep (fast path)
    int ndir;          // sweeps per sample in the tile kernel: always two, which bracket the result (see sweep_tiles_group)
    // The two tile sweeps of a sample: direction (0: alpha, 1: beta) and rounding side (0: every number too small
    // for the linear domain becomes 0, a lower bound of the sum over paths; 1: it becomes the smallest number the
    // domain holds, an upper bound).  With gradients {alpha/upper, beta/lower}, without {alpha/lower, alpha/upper}.
    unsigned char rev[2], upper[2];
    int only_flagged;  // exact kernel: 0 = every sample; 1 = samples whose flag is set
    unsigned char gtab[kMaxBlocksFast + 1][12];  // fast path: gtab[NBb][g] = first block of group g (host-built)
    double *zfast;     // [2][B] the fast kernel's own read-outs (never rewritten by the exact kernel)
};

__device__ __forceinline__ bool lengths_ok(int Lb, int Tb, int L, int T) {
    return Tb >= 1 && Lb >= 1 && Tb <= T && Lb <= L && Tb <= Lb;
}

// A chunk of R terms held in registers, merged into (m,s): max pass, then exp-sum pass.  The terms and the
// running maximum are float64 (absolute log values of any magnitude),
// the exponentials of the differences and their sum float32.
template <int R>
__device__ __forceinline__ void lse_chunk_d(const double (&x)[R], double &m, float &s) {
    double cm = x[0];
#pragma unroll
    for (int r = 1; r < R; ++r) cm = fmax(cm, x[r]);
    if (cm == (double)DAGX_NEG_INF) {   // nothing finite here (fmax skips a NaN, which must not get lost)
        bool nan = false;
#pragma unroll
        for (int r = 0; r < R; ++r) nan |= x[r] != x[r];
        if (nan) s = __builtin_nanf("");
        return;
    }
    const double nm = fmax(m, cm);
    float part = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) part += fast_exp2((float)(x[r] - nm) * kLog2e);
    s = s * fast_exp2((float)(m - nm) * kLog2e) + part;  // m = -inf gives 0 * 0
    m = nm;
}

__device__ __forceinline__ double wave_max_d(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmax(v, __shfl_xor(v, o, kWave));
    return v;
}

// ================================================================================================
// Exact sweep
// ================================================================================================

// One row of the table from this step's values by node (absolute, float64): per block of 64 positions the
// offset is the block maximum and the residuals are what is left, so that no cell's precision depends on
// how far it lies under the largest value of the row.
template <int NT>
__device__ __forceinline__ void write_row(const double *f, int dir, int Lb, int NBb, float *hat_row, double *off_row) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    for (int blk = wave; blk < NBb; blk += NT / kWave) {
        const int p = blk * kBlk + lane;
        const int node = dir ? Lb - 1 - p : p;
        const double v = p < Lb ? f[node] : (double)DAGX_NEG_INF;
        const double bm = wave_max_d(v);
        if (lane == 0) off_row[blk] = bm;
        if (p < Lb) hat_row[node] = bm > (double)DAGX_NEG_INF ? (float)(v - bm) : DAGX_NEG_INF;
    }
}

// Log-domain sweeps, one workgroup per (sample, direction).  The running vector is kept in float64 (LDS), every
// term is formed as a float64 sum and only the difference to the cell's own running maximum is exponentiated
// in float32: cells hundreds or thousands of nats under the largest value of their step, which is where the
// posterior mass of sharply peaked inputs can sit, keep the full precision of their inputs.
template <typename TM, typename TL, int NT>
__device__ __forceinline__ void exact_sweep_sample(const SweepArgs &a, const int b, const int dir, double *lds_x) {
    // lds_x: two vectors of L doubles;  dir 0: alpha, 1: beta
    const int tid = threadIdx.x;
    const int L = a.L, T = a.T, translen = a.translen;
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
    const TM *match = static_cast<const TM *>(a.match) + (int64_t)b * a.ms0;
    const TL *links = static_cast<const TL *>(a.links) + (int64_t)b * L * translen;
    float *hat = a.hat[dir] + (int64_t)b * T * L;
    double *off = a.off[dir] + (int64_t)b * T * a.NBK;
    double *fprev = lds_x, *fcur = lds_x + L;

    if (!lengths_ok(Lb, Tb, L, T)) {
        if (tid == 0) { a.logz[dir * a.B + b] = (double)DAGX_NEG_INF; if (dir == a.loss_dir) a.loss[b] = DAGX_NEG_INF; }
        return;
    }
    const int slack = Lb - Tb;  // band: s <= p <= slack + s
    const int NBb = (Lb + kBlk - 1) / kBlk;
    const int t0 = dir ? Tb - 1 : 0, start = dir ? Lb - 1 : 0;
    const float m0 = to_float(match[(int64_t)t0 * a.ms1 + (int64_t)start * a.ms2]);
    for (int j = tid; j < L; j += NT) fprev[j] = j == start ? (double)m0 : (double)DAGX_NEG_INF;
    __syncthreads();
    write_row<NT>(fprev, dir, Lb, NBb, hat + (int64_t)t0 * L, off + (int64_t)t0 * a.NBK);

    // A team of kTeam lanes works on one node; each of its lanes has R terms in flight.
    constexpr int kTeam = 8, R = 8;
    const int team = tid / kTeam, sub = tid % kTeam;
    auto team_merge = [](double &m, float &sum) {   // the lanes' (maximum, sum) pairs into one, in every lane of the team
#pragma unroll
        for (int o = kTeam / 2; o > 0; o >>= 1) {
            const double mo = __shfl_xor(m, o, kWave);
            const float so = __shfl_xor(sum, o, kWave);
            const double nm = fmax(m, mo);
            if (nm > (double)DAGX_NEG_INF)
                sum = sum * fast_exp2((float)(m - nm) * kLog2e) + so * fast_exp2((float)(mo - nm) * kLog2e);
            else
                sum += so;   // 0 + 0, or a NaN on its way
            m = nm;
        }
    };
    for (int s = 1; s < Tb; ++s) {
        const int t = dir ? Tb - 1 - s : s;
        if (dir == 0) {
            // A team of kTeam lanes <-> node j of the band; the team's lanes deal the predecessors i among
            // themselves (lane q takes i = ilo + q, ilo + q + kTeam, ...), R of them in flight per lane, and
            // merge their (maximum, sum) pairs by shuffles.  Teams of one wave hold neighbouring nodes, so a
            // wave-wide load reads kTeam runs of neighbouring elements; nodes are dealt to the teams round
            // robin, which mixes nodes with few and with many predecessors in every team.
            const int jhi = slack + s;
            for (int j = tid; j < L; j += NT)
                if (j < s || j > jhi) fcur[j] = (double)DAGX_NEG_INF;
            const unsigned rs = (unsigned)(translen - 1);   // E[i][j-i-1] sits at links[i*(translen-1) + j-1]: 32-bit offsets
            for (int j = s + team; j <= jhi; j += NT / kTeam) {
                const float mj = to_float(match[(int64_t)t * a.ms1 + (int64_t)j * a.ms2]);
                int ilo = j - translen; if (ilo < s - 1) ilo = s - 1;
                double m = (double)DAGX_NEG_INF; float sum = 0.f;
                const unsigned o_last = (unsigned)(j - 1) * (unsigned)translen;   // the offset of i = j-1, the largest
                unsigned o = (unsigned)(ilo + sub) * rs + (unsigned)(j - 1);
                for (int i0 = ilo + sub; i0 < j; i0 += kTeam * R, o += kTeam * R * rs) {
                    float e[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const unsigned oc = o + (unsigned)(r * kTeam) * rs;
                        e[r] = to_float(links[oc < o_last ? oc : o_last]);
                    }
                    double x[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) {   // a term beyond the last predecessor: -inf through its transition
                        const int i = i0 + r * kTeam;
                        x[r] = fprev[i < j ? i : j - 1] + (double)(i < j ? e[r] : DAGX_NEG_INF);
                    }
                    lse_chunk_d<R>(x, m, sum);
                }
                team_merge(m, sum);
                if (sub == 0)
                    fcur[j] = (m > (double)DAGX_NEG_INF || sum != sum) ? (m + (double)(fast_log2(sum) * kLn2)) + (double)mj : (double)DAGX_NEG_INF;
            }
        } else {
            // the same with a team <-> node i and the team's lanes dealing the successors j among themselves: a
            // team reads runs of kTeam neighbouring elements of its node's row of links
            const int ilo_band = Lb - 1 - (slack + s), ihi_band = Lb - 1 - s;  // nodes whose position is in the band
            const int jtop = Lb - 1 - (s - 1), jbot = Lb - 1 - (slack + s - 1);  // band of the previous step
            for (int i = tid; i < L; i += NT)
                if (i < ilo_band || i > ihi_band) fcur[i] = (double)DAGX_NEG_INF;
            for (int i = ilo_band + team; i <= ihi_band; i += NT / kTeam) {
                const float mi = to_float(match[(int64_t)t * a.ms1 + (int64_t)i * a.ms2]);
                const int jmax = i + translen < jtop ? i + translen : jtop;
                const int jmin = i + 1 > jbot ? i + 1 : jbot;
                const unsigned rbase = (unsigned)i * (unsigned)translen - (unsigned)i - 1u;   // E[i][j-i-1] = links[rbase + j], modulo 2^32
                double m = (double)DAGX_NEG_INF; float sum = 0.f;
                for (int j0 = jmin + sub; j0 <= jmax; j0 += kTeam * R) {
                    float e[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const int j = j0 + r * kTeam;
                        e[r] = to_float(links[rbase + (unsigned)(j <= jmax ? j : jmax)]);
                    }
                    double x[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const int j = j0 + r * kTeam;
                        x[r] = fprev[j <= jmax ? j : jmax] + (double)(j <= jmax ? e[r] : DAGX_NEG_INF);
                    }
                    lse_chunk_d<R>(x, m, sum);
                }
                team_merge(m, sum);
                if (sub == 0)
                    fcur[i] = (m > (double)DAGX_NEG_INF || sum != sum) ? (m + (double)(fast_log2(sum) * kLn2)) + (double)mi : (double)DAGX_NEG_INF;
            }
        }
        __syncthreads();
        write_row<NT>(fcur, dir, Lb, NBb, hat + (int64_t)t * L, off + (int64_t)t * a.NBK);
        double *sw = fprev; fprev = fcur; fcur = sw;
    }
    if (tid == 0) {
        const double z = fprev[dir ? 0 : Lb - 1];
        a.logz[dir * a.B + b] = z;
        if (dir == a.loss_dir) a.loss[b] = (float)z;
    }
}

template <typename TM, typename TL, int NT>
__global__ __launch_bounds__(NT) void dag_sweep_exact_kernel(SweepArgs a) {
    extern __shared__ double lds_x[];
    if (a.only_flagged && a.flags[blockIdx.x] != 1) return;
    exact_sweep_sample<TM, TL, NT>(a, (int)blockIdx.x, (int)blockIdx.y, lds_x);
}

// ================================================================================================
// Fast sweep: register-resident exp(E) tiles, DPP broadcast FMAs, pipelined workgroups
// ================================================================================================

// One step of one tile: sum_r e[r] * P[r][lane], e given 16-replicated in four registers
__device__ __forceinline__ float tile_dot(const Tile &t, float e0, float e1, float e2, float e3) {
    // one accumulator, started by a multiply: dependent DPP FMAs issue as fast as independent ones here, and
    // every instruction saved is an issue slot of the SIMD
    float a;
    mul16_rowbcast(a, e0, t.p);
    fma16_rowbcast(a, e1, t.p + 16);
    fma16_rowbcast(a, e2, t.p + 32);
    fma16_rowbcast(a, e3, t.p + 48);
    return a;
}

// ---- the wide variant: the same sweep with float64 linear-domain numbers --------------------------------------
// What the float32 sweep cannot hold is, almost always, a cell far under the maximum of its block or a block far
// under its neighbours (inputs whose best prefixes are not the prefixes of the best paths); a float64 number has
// room for 1300 nats under its scale where a float32 number has 126.  The wide variant keeps exp(residual), the
// tile sums, the block factors and their sums in float64; the staged transitions stay float32 registers (the
// register file holds no float64 tiles) and are converted as they are used: v_cvt_f64_f32 + v_fmac_f64 with the
// same DPP row broadcast, two instructions per pair-update instead of one.  It runs, as a second launch, on the
// samples whose float32 sweeps did not agree, and leaves to the log-domain kernel what it cannot settle either.
constexpr int kShiftWide = 850;   // float64 numbers carry 2^850: 2^(850 + 127 + 10) < 2^1024 above, 2^-1022 below

// acc += sum_{r<16} e[lane r of this lane's 16-lane row] * (double)p[r]
__device__ __forceinline__ void fma16_rowbcast(double &acc, double e, const float *p) {
    double t0, t1;
    asm("s_nop 1\n\t"
        "v_cvt_f64_f32 %1, %4\n\t"
        "v_cvt_f64_f32 %2, %5\n\t"
        "v_fmac_f64_dpp %0, %3, %1 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %1, %6\n\t"
        "v_fmac_f64_dpp %0, %3, %2 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %2, %7\n\t"
        "v_fmac_f64_dpp %0, %3, %1 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %1, %8\n\t"
        "v_fmac_f64_dpp %0, %3, %2 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %2, %9\n\t"
        "v_fmac_f64_dpp %0, %3, %1 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %1, %10\n\t"
        "v_fmac_f64_dpp %0, %3, %2 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %2, %11\n\t"
        "v_fmac_f64_dpp %0, %3, %1 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %1, %12\n\t"
        "v_fmac_f64_dpp %0, %3, %2 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %2, %13\n\t"
        "v_fmac_f64_dpp %0, %3, %1 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %1, %14\n\t"
        "v_fmac_f64_dpp %0, %3, %2 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %2, %15\n\t"
        "v_fmac_f64_dpp %0, %3, %1 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %1, %16\n\t"
        "v_fmac_f64_dpp %0, %3, %2 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %2, %17\n\t"
        "v_fmac_f64_dpp %0, %3, %1 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %1, %18\n\t"
        "v_fmac_f64_dpp %0, %3, %2 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
        "v_cvt_f64_f32 %2, %19\n\t"
        "v_fmac_f64_dpp %0, %3, %1 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_fmac_f64_dpp %0, %3, %2 row_newbcast:15 row_mask:0xf bank_mask:0xf"
        : "+v"(acc), "=&v"(t0), "=&v"(t1)
        : "v"(e), "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]),
          "v"(p[8]), "v"(p[9]), "v"(p[10]), "v"(p[11]), "v"(p[12]), "v"(p[13]), "v"(p[14]), "v"(p[15]));
}
__device__ __forceinline__ double tile_dot(const Tile &t, double e0, double e1, double e2, double e3) {
    double a = 0.0;
    fma16_rowbcast(a, e0, t.p);
    fma16_rowbcast(a, e1, t.p + 16);
    fma16_rowbcast(a, e2, t.p + 32);
    fma16_rowbcast(a, e3, t.p + 48);
    return a;
}
// the same with the tile's last NT rows held elsewhere
template <int NT>
__device__ __forceinline__ double tile_dot_tail(const Tile &t, const float (&tail)[NT], double e0, double e1, double e2, double e3) {
    static_assert(NT > 0 && NT <= 16, "");
    float last[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) last[u] = u < 16 - NT ? t.p[48 + u] : tail[u - (16 - NT)];
    double a = 0.0;
    fma16_rowbcast(a, e0, t.p);
    fma16_rowbcast(a, e1, t.p + 16);
    fma16_rowbcast(a, e2, t.p + 32);
    fma16_rowbcast(a, e3, last);
    return a;
}
template <int U0>
__device__ __forceinline__ void scaled_sum4(double &acc, double f, double v0, double v1, double v2, double v3) {
    static_assert(U0 % 4 == 0 && U0 >= 0 && U0 < 16, "");
    if constexpr (U0 == 0) acc = 0.0;
    asm("s_nop 1\n\t"
        "v_fmac_f64_dpp %0, %1, %2 row_newbcast:%c6 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %0, %1, %3 row_newbcast:%c7 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %0, %1, %4 row_newbcast:%c8 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f64_dpp %0, %1, %5 row_newbcast:%c9 row_mask:0xf bank_mask:0xf"
        : "+v"(acc) : "v"(f), "v"(v0), "v"(v1), "v"(v2), "v"(v3), "n"(U0), "n"(U0 + 1), "n"(U0 + 2), "n"(U0 + 3));
}

// The linear-domain number type of a sweep and what depends on it.
template <bool WIDE> struct Lin;
template <> struct Lin<false> {
    using T = float;
    static constexpr float kFacFloor = -126.f;                       // upper sweep: smallest exponent of a block factor
    __device__ static __forceinline__ float tiny() { return kTinyStored; }
    __device__ static __forceinline__ float flushed_sum() { return 2.4074124e-35f; }   // 2^-115, see own_block
    __device__ static __forceinline__ float exp2s(float x) { return exp2_shifted(x); }          // 2^(x + shift)
    __device__ static __forceinline__ float exp2u(float x) { return fast_exp2(x); }             // 2^x
    __device__ static __forceinline__ float log2u(float y) { return log2_unshifted(y); }        // log2(y) - 2 * shift
};
template <> struct Lin<true> {
    using T = double;
    static constexpr float kFacFloor = -1022.f;
    __device__ static __forceinline__ double tiny() { return 2.2250738585072014e-308; }          // 2^-1022
    __device__ static __forceinline__ double flushed_sum() { return 9.332636185032189e-302; }    // 2^-1000
    // 2^(x + shift) for a float x (any value; -inf gives 0, a NaN stays one): the fraction through v_exp_f32, the
    // integer part through the exponent field
    __device__ static __forceinline__ double exp2_with(float x, int shift) {
        const float n = __builtin_floorf(x);
        const double m = (double)fast_exp2(x - n);
        const double r = __builtin_ldexp(m, (int)__builtin_fmaxf(n, -4000.f) + shift);
        return !(x <= -3000.f) ? r : 0.0;
    }
    // the same for a float64 argument (scale arithmetic of the wide sweeps: differences of offsets hundreds of nats
    // apart, whose float32 rounding, repeated every step, would add up along a path)
    __device__ static __forceinline__ double exp2_with(double x, int shift) {
        const double n = __builtin_floor(x);
        const double m = (double)fast_exp2((float)(x - n));
        const double r = __builtin_ldexp(m, (int)(n > -4000.0 ? n : -4000.0) + shift);
        return !(x <= -3000.0) ? r : 0.0;
    }
    // y * 2^x with the integer part of x going into y's exponent field (2^x by itself may lie outside the float64
    // range where the product does not); x = -inf gives 0
    __device__ static __forceinline__ double times_exp2(double y, double x) {
        const double n = __builtin_floor(x);
        const double m = (double)fast_exp2((float)(x - n));
        const double r = __builtin_ldexp(y * m, (int)(n > -8000.0 ? n : -8000.0));
        return !(x <= -6000.0) ? r : 0.0;
    }
    __device__ static __forceinline__ double exp2s(float x) { return exp2_with(x, kShiftWide); }
    __device__ static __forceinline__ double exp2u(float x) { return exp2_with(x, 0); }
    // log2(y) minus the shift of a float64 number and that of a staged transition
    __device__ static __forceinline__ float log2u(double y) {
        return (float)(__builtin_amdgcn_frexp_exp(y) - (kShiftWide + kShiftLinksWide)) + fast_log2((float)__builtin_amdgcn_frexp_mant(y));
    }
    // the same as a float64 number: the exponent exactly, the logarithm of the fraction (in [-1, 0]) from v_log_f32
    __device__ static __forceinline__ double log2u_wide(double y) {
        return (double)(__builtin_amdgcn_frexp_exp(y) - (kShiftWide + kShiftLinksWide)) + (double)fast_log2((float)__builtin_amdgcn_frexp_mant(y));
    }
};

constexpr int kPartBlocks = 12;   // a group never owns more blocks: every block but the first has >= 2 tiles
constexpr int kPartRows = 16;     // partial-sum rows reserved per owned block (tiles per block <= 16)
// LDS of the step loop.  First the linear-domain numbers, indexed in elements of the sweep's number type:
constexpr int kEvEbuf = 0;                                              // [2][16][64] exp(residual), by position
constexpr int kEvPart = kEvEbuf + 2 * kMaxBlocksFast * kBlk;            // [12][16][64] per-tile partial sums
constexpr int kEvNowhere = kEvPart + kPartBlocks * kPartRows * kBlk;    // [64] where a wave's unused tile slots "write their partial sums"
constexpr int kEvCount = kEvNowhere + kBlk;
// then, in floats from the start of the dynamic segment:
template <bool WIDE> struct StepLds {
    static constexpr int kRelb = kEvCount * (WIDE ? 2 : 1);              // [2][16] block offsets rel. to the reference (float; double in the wide variant)
    // landing areas of the asynchronous global -> LDS copies (one slot per consuming wave), double-buffered by step parity
    static constexpr int kStageM = kRelb + 2 * kMaxBlocksFast * (WIDE ? 2 : 1);   // [2][8 waves][2][64] dwords: match rows of each wave's own blocks (raw elements)
    static constexpr int kStageF = kStageM + 2 * kTileWaves * 2 * kBlk;  // [2][8 waves][2][64] floats: table residuals of the wave's foreign blocks
    static constexpr int kStageO = kStageF + 2 * kTileWaves * 2 * kBlk;  // [2][64] dwords: the table's offset row (16 doubles, padded)
    static constexpr int kStageP = kStageO + 2 * kBlk;                    // [2][64] dwords: snapshot of the progress word of the group below
    static constexpr int kLastV = kStageP + 2 * kBlk;                    // [8 waves][64] the values of the last step (for the read-out)
    static constexpr int kLastC = kLastV + kTileWaves * kBlk * (WIDE ? 2 : 1);   // [8 waves] doubles: the reference they are relative to
    // (kLastV holds float64 values in the wide variant: twice the room)
    // the wide variant keeps the last rows of every wave's third tile here and reads them back in every step: the
    // registers they would occupy are what its float64 temporaries of phase B need
    static constexpr int kTailRows = WIDE ? 12 : 0;
    static constexpr int kTail = kLastC + 2 * kTileWaves;                // [8 waves][kTailRows][64] floats
    static constexpr int kStepFloats = kTail + kTileWaves * kTailRows * kBlk;
};

// Memory traffic of the loop is asynchronous and off the critical path.  The last wave of the
// workgroup is the fetcher (it holds no tiles whenever the group has at most 21): during phase A of
// step s, while the other waves run their tiles, it requests (global -> LDS copies) what phase B of step
// s + 1 needs -- the match rows of every owned block and, for consumer groups, the table rows of the
// foreign blocks and a snapshot of the producer's progress word -- and only waits for what it requested
// a whole step earlier.  Nobody waits for a load that was issued in the same step, unless a consumer
// has caught up with its producer; then the fetcher polls the progress word (bounded).
//
// Inter-workgroup hand-over of the running vector (groups of one sweep form a one-way pipeline):
//  * a producer writes its table rows (hat, off) with agent-scope write-through stores; a step
//    later, when every wave has seen those stores complete, it raises its progress word;
//  * a consumer's fetcher copies the rows of a step once a snapshot of that word covers the step.
// Every wait is bounded: on expiry the sample is marked for the exact kernel and the group leaves.
//
// Leaving: every workgroup counts itself out of its sample and out of the launch.  The last one of a
// sample compares the two read-outs of the tile sweeps, sets the sample's flag (1 = the log-domain kernel
// must redo it) and clears the sample's pipeline words; the last one of the launch clears the ticket
// counter -- so the words are all zero again when the launch is over and need no fill in front of it.
//
// The step loop is issue-bound (two waves per SIMD, a few hundred instructions per wave and step
// around the 64 FMAs of each tile), so everything that does not change from step to step -- LDS
// addresses, table offsets, the tile's band limits -- is computed before the loop, the loop body is
// instantiated for both parities of the double buffers (immediate LDS offsets), and the LDS reads
// of a phase are issued together.
template <typename TM, typename TL, bool WIDE>
__device__ __forceinline__ void sweep_tiles_group(const SweepArgs &a, const int b, const int slot, const int g, float *lds_raw,
                                                  int *gstart, int *s_abort_p) {
    using LN = Lin<WIDE>;
    using EV = typename LN::T;          // exp(residual), tile sums, block factors: float, or double in the wide variant
    // A cell's value relative to the step's reference: float, or double in the wide variant -- its samples are the
    // ones whose values lie hundreds of nats from their reference, where a float32 value is 3e-5 coarse, and the
    // two read-outs of a sample can only be held to 5e-5 of each other if they are finer than that.
    using VT = typename LN::T;
    using LD = StepLds<WIDE>;
    constexpr int kLdsRelb = LD::kRelb, kLdsStageM = LD::kStageM, kLdsStageF = LD::kStageF, kLdsStageO = LD::kStageO,
                  kLdsStageP = LD::kStageP, kLdsLastV = LD::kLastV, kLdsLastC = LD::kLastC, kLdsStepFloats = LD::kStepFloats;
    // slot: which of the sample's two sweeps (its tables, pipeline words and read-out); dir: its direction;
    // upper: its rounding side.  The linear domain flushes what is more than 126 nats under its scale -- a
    // transition, a cell under its block maximum, a block under the largest of its neighbours, a product of such
    // numbers.  The lower sweep lets all of that become 0, so its read-out never exceeds log Z; the upper sweep
    // puts the smallest normal number (or a constant that covers every flushed product) in its place, so its
    // read-out never falls short of log Z.  The sample's result stands when the two read-outs agree; what was
    // flushed then carried no mass that matters, wherever it was flushed.
    const int dir = a.rev[slot];
    const bool upper = a.upper[slot] != 0;
    // Dynamic LDS, used twice: while the tiles are staged it holds one transpose patch per wave
    // ([kTileWaves][kBlk][kBlk+1], beta tiles only); after the barrier that ends staging it holds the
    // step buffers (kLds* above).
    float (*stage)[kBlk][kBlk + 1] = reinterpret_cast<float (*)[kBlk][kBlk + 1]>(lds_raw);
    int &s_abort = *s_abort_p;
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int C = a.C;
    int *risk = a.sync + 16 + a.ndir * a.B * C + a.B + b;

    // (taken through opaque_uniform: otherwise the compiler re-reads them from the argument block inside the
    //  step loop, a scalar-memory round trip on the critical path, instead of keeping them in registers)
    const int L = opaque_uniform(a.L), T = a.T, translen = a.translen, NBK = opaque_uniform(a.NBK);
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
    if (!lengths_ok(Lb, Tb, L, T)) {
        if (g == 0 && tid == 0) { a.logz[slot * a.B + b] = (double)DAGX_NEG_INF; if (slot == a.loss_dir) a.loss[b] = DAGX_NEG_INF; store_agent(a.zfast + slot * a.B + b, (double)DAGX_NEG_INF); }
        return;
    }
    const TM *match = static_cast<const TM *>(a.match) + (int64_t)b * a.ms0;
    const TL *links = static_cast<const TL *>(a.links) + (int64_t)b * L * translen;
    float *hat = a.hat[slot] + (int64_t)b * T * L;
    double *off = a.off[slot] + (int64_t)b * T * NBK;
    int *prog = a.sync + 16 + (slot * a.B + b) * C;

    const int slack = Lb - Tb;
    const int NBb = (Lb + kBlk - 1) / kBlk;
    const int W = (translen + kBlk - 1) / kBlk;
    if (tid <= C) gstart[tid] = a.gtab[NBb][tid];
    __syncthreads();
    const int jb0 = __builtin_amdgcn_readfirstlane(gstart[g]), jb1 = __builtin_amdgcn_readfirstlane(gstart[g + 1]);
    int last_group = 0;
    for (int q = 0; q < C; ++q) if (gstart[q + 1] > gstart[q]) last_group = q;
    last_group = __builtin_amdgcn_readfirstlane(last_group);
    if (jb0 >= jb1) return;  // nothing to do for this group (short sample); nobody waits on it
    const int nblk = jb1 - jb0;
    const int flo = tile_ilo(jb0, W);  // lowest foreign block this group ever reads
    const bool producer = g < last_group;
    const bool unlimited = W >= NBb - 1;   // every lower block is a predecessor block
    if (nblk > kPartBlocks) {  // cannot happen with the host's partition; leave the sample to the exact kernel
        if (tid == 0) { store_agent(risk, 1); store_agent(prog + g, 1 << 30); }
        return;
    }

    // ---- my tiles: enumerated block by block; each wave takes a contiguous run of them ----
    int ntile = 0;
    for (int Jb = jb0; Jb < jb1; ++Jb) ntile += Jb - tile_ilo(Jb, W) + 1;
    // The last wave fetches (see above) and takes tiles only when the others cannot hold them all.  The
    // tiles are dealt out evenly; the odd ones go first to wave 3, whose SIMD it shares with the
    // fetcher, then to waves 0, 1, 2, 4, ...
    const int nwork = ntile <= kTilesPerWave * (kTileWaves - 1) ? kTileWaves - 1 : kTileWaves;
    int my_first = 0, my_count = 0;
    {
        const int base = ntile / nwork, rem = ntile % nwork;
        int first = 0;
        for (int w = 0; w < kTileWaves; ++w) {
            const int rank = nwork == kTileWaves ? w : (w == 3 ? 0 : (w < 3 ? w + 1 : w));
            const int cnt = w < nwork ? base + (rank < rem ? 1 : 0) : 0;
            if (w == wave) { my_first = first; my_count = cnt; }
            first += cnt;
        }
    }
    int my_I[kTilesPerWave], my_J[kTilesPerWave];
    bool my_ok[kTilesPerWave];
#pragma unroll
    for (int sl = 0; sl < kTilesPerWave; ++sl) { my_I[sl] = 0; my_J[sl] = jb0; my_ok[sl] = false; }
    {
        int q = 0;
        for (int Jb = jb0; Jb < jb1; ++Jb)
            for (int I = tile_ilo(Jb, W); I <= Jb; ++I, ++q) {
                const int sl = q - my_first;
                if (sl >= 0 && sl < my_count) {
#pragma unroll
                    for (int u = 0; u < kTilesPerWave; ++u)
                        if (u == sl) { my_I[u] = I; my_J[u] = Jb; my_ok[u] = true; }
                }
            }
    }
    Tile t0, t1, t2;
    // What a finite transition below the staged range becomes: 0 in a lower sweep, the smallest number the staged
    // range holds in an upper sweep (exp(-126) under a certain transition in the float32 sweeps, exp(-175) in the
    // wide ones).
    constexpr int kLinkShift = WIDE ? kShiftLinksWide : kShift2;
    const float tiny = !upper ? 0.f : kTinyStored;   // (2^-126 as stored: at least any transition that is not staged, in either variant)
    if (my_ok[0]) load_tile<true, 16, TL, kLinkShift>(t0, links, my_I[0], my_J[0], lane, dir, Lb, translen, stage[wave], tiny);
    if (my_ok[1]) load_tile<true, 16, TL, kLinkShift>(t1, links, my_I[1], my_J[1], lane, dir, Lb, translen, stage[wave], tiny);
    if (my_ok[2]) load_tile<true, 16, TL, kLinkShift>(t2, links, my_I[2], my_J[2], lane, dir, Lb, translen, stage[wave], tiny);
    __syncthreads();   // every wave is done with its transpose patch: the LDS now holds the step buffers

    EV *const ebuf = reinterpret_cast<EV *>(lds_raw) + kEvEbuf;   // [parity][block][64]
    float *const relb = lds_raw + kLdsRelb;   // [parity][block]
    double *const relb64 = reinterpret_cast<double *>(lds_raw + kLdsRelb);   // the same in the wide variant
    constexpr int kEbufPar = kMaxBlocksFast * kBlk;   // floats between the two parities of ebuf

    // ---- step 0 is known to every group: only position 0 is alive ----
    const int t_first = dir ? Tb - 1 : 0, node_first = dir ? Lb - 1 : 0;
    const float m0 = to_float(match[(int64_t)t_first * a.ms1 + (int64_t)node_first * a.ms2]);
    const bool alive0 = m0 > DAGX_NEG_INF;
    double cref = alive0 ? (double)m0 : 0.0;  // absolute value the relb / v numbers of this step are relative to
    for (int q = tid; q < kLdsStepFloats; q += kTileWaves * kWave) lds_raw[q] = 0.f;   // ebuf, part (rows no tile writes stay 0)
    __syncthreads();
    constexpr int kTailRows = LD::kTailRows, kTailFirst = kBlk - kTailRows;
    float *const tail_lane = lds_raw + LD::kTail + wave * (kTailRows * kBlk) + lane;   // (read and written by this wave alone)
    if constexpr (WIDE) {
#pragma unroll
        for (int u = 0; u < kTailRows; ++u) tail_lane[u * kBlk] = my_ok[2] ? t2.p[kTailFirst + u] : 0.f;
    }
    if (tid == 0 && alive0) ebuf[0] = LN::exp2s(0.f);
    if (tid < 2 * kMaxBlocksFast) {
        if constexpr (WIDE) relb64[tid] = (tid == 0 && alive0) ? 0.0 : (double)DAGX_NEG_INF;
        else relb[tid] = (tid == 0 && alive0) ? 0.f : DAGX_NEG_INF;
    }
    for (int ob = wave; ob < nblk; ob += kTileWaves) {  // own blocks of the first row of the table
        const int Jb = jb0 + ob, p = Jb * kBlk + lane;
        if (p < Lb) store_agent(hat + (int64_t)t_first * L + (dir ? Lb - 1 - p : p), (p == 0 && alive0) ? 0.f : DAGX_NEG_INF);
        if (lane == 0) store_agent(off + (int64_t)t_first * NBK + Jb, (Jb == 0 && alive0) ? (double)m0 : (double)DAGX_NEG_INF);
    }
    if (Tb == 1 && tid == 0 && jb0 == 0) {
        const double z = (Lb == 1 && alive0) ? (double)m0 : (double)DAGX_NEG_INF;
        a.logz[slot * a.B + b] = z; if (slot == a.loss_dir) a.loss[b] = (float)z; store_agent(a.zfast + slot * a.B + b, z);
    }

    // Table rows are addressed as (uniform base) + 32-bit byte offset so that no 64-bit per-lane
    // addresses stay live across the step loop (every register is needed for the tiles).
    const char *hat_c = reinterpret_cast<const char *>(hat);
    const char *off_c = reinterpret_cast<const char *>(off);
    const char *match_c = reinterpret_cast<const char *>(match);
    auto hat_at = [&](int trow, int node) -> float * {
        return reinterpret_cast<float *>(const_cast<char *>(hat_c) + (unsigned)(trow * L + node) * 4u);
    };
    auto off_at = [&](int trow, int blk) -> double * {
        return reinterpret_cast<double *>(const_cast<char *>(off_c) + (unsigned)(trow * NBK + blk) * 8u);
    };
    const int ms1 = (int)a.ms1, ms2 = (int)a.ms2;   // the host checked that match indices fit 32 bits

    // ---- loop invariants of this wave ----
    // Wave-uniform element offsets into the LDS (kept in scalar registers; per-lane addresses are
    // formed from them inside the loop -- there is no vector register to spare for them):
    // where a tile reads its e values and writes its partial sum, and the steps at which its output
    // block lies inside the band (s_lo <= s <= s_hi).
    int e_off[kTilesPerWave], part_off[kTilesPerWave], s_lo[kTilesPerWave], s_hi[kTilesPerWave];
#pragma unroll
    for (int sl = 0; sl < kTilesPerWave; ++sl) {
        e_off[sl] = __builtin_amdgcn_readfirstlane(kEvEbuf + my_I[sl] * kBlk);
        part_off[sl] = __builtin_amdgcn_readfirstlane(kEvPart + ((my_J[sl] - jb0) * kPartRows + (my_I[sl] - tile_ilo(my_J[sl], W))) * kBlk);
        s_lo[sl] = __builtin_amdgcn_readfirstlane(my_J[sl] * kBlk - slack);
        s_hi[sl] = __builtin_amdgcn_readfirstlane(my_J[sl] * kBlk + kBlk - 1);
        // a slot without a tile is never "in the band" and stores its zero where nobody reads: no test of its own
        // in the loop (every test there is an instruction slot, and its operands live in scarce scalar registers)
        if (!my_ok[sl]) { part_off[sl] = kEvNowhere; s_lo[sl] = 0x7fffffff; s_hi[sl] = -1; }
    }
    const float fac_floor = upper ? LN::kFacFloor : DAGX_NEG_INF;
    // The direction of rounding as numbers, not as a condition (a wave-uniform condition is a pair of scalar registers,
    // and the loop has none to spare: it came back from a vector register's lanes at every use): what a flushed live
    // cell becomes, and what is added to every block sum for the products that may have been flushed.
    EV tiny_up = upper ? LN::tiny() : (EV)0, flush_up = upper ? LN::flushed_sum() : (EV)0;
    asm volatile("" : "+v"(tiny_up), "+v"(flush_up));
    const float *const lds_l15 = lds_raw + (lane & 15);   // every 16-lane row addresses the same 16 values
    float *const lds_lane = lds_raw + lane;
    const EV *const ev_l15 = reinterpret_cast<const EV *>(lds_raw) + (lane & 15);   // the same two for the linear-domain numbers
    EV *const ev_lane = reinterpret_cast<EV *>(lds_raw) + lane;
    // the block this wave owns in phase B (a second one, wave + 8, is handled without look-ahead)
    const bool owner = wave < nblk;
    const int Jown = jb0 + (owner ? wave : 0);
    const int p_own = Jown * kBlk + lane;
    const int node_own = dir ? Lb - 1 - p_own : p_own;
    const int nt_own = Jown - tile_ilo(Jown, W) + 1;
    const int own_part_off = __builtin_amdgcn_readfirstlane(kEvPart + (owner ? wave : 0) * kPartRows * kBlk);
    // ---- staging slots: the match rows of own blocks wave and wave + 8, the table rows of two foreign blocks
    //      (converted by this wave in phase B; dealt from the last wave down, so that the first waves, which own
    //      blocks, rarely have a conversion in front of their own block's chain of dependent steps), one offset row ----
    const unsigned lds_base = (unsigned)reinterpret_cast<uintptr_t>(lds_raw);   // LDS byte address of the dynamic segment
    constexpr int kFetchSlots = 2;
    const bool consumer = flo < jb0;
    int f_blk[kFetchSlots];
#pragma unroll
    for (int u = 0; u < kFetchSlots; ++u) {
        const int fb = flo + (kTileWaves - 1 - wave) + kTileWaves * u;
        f_blk[u] = fb < jb0 ? fb : -1;
    }
    const int *below = prog + (g > 0 ? g - 1 : 0);
    auto stage_m_of = [&](int par, int w, int u) -> int { return kLdsStageM + ((par * kTileWaves + w) * 2 + u) * kBlk; };
    auto stage_f_of = [&](int par, int w, int u) -> int { return kLdsStageF + ((par * kTileWaves + w) * 2 + u) * kBlk; };
    auto stage_m = [&](int par, int u) -> int { return stage_m_of(par, wave, u); };
    auto stage_f = [&](int par, int u) -> int { return stage_f_of(par, wave, u); };
    auto stage_o = [&](int par) -> int { return kLdsStageO + par * kBlk; };
    auto stage_p = [&](int par) -> int { return kLdsStageP + par * kBlk; };
    // ---- the fetcher (last wave): everything phase B reads from memory, requested one step ahead ----
    const bool fetcher = wave == kTileWaves - 1;
    int seen = 0;          // latest progress value of the group below known to the fetcher
    int rows_issued = 0;   // the foreign table rows of steps <= rows_issued have been requested
    int snapshot = 0;      // the producer's progress word as copied a step ago: what every wave of the group acts on
    // A copy's address is (scalar base of the row and block) + (per-lane offset inside a block, the same for
    // every block, recomputed each step from the lane number: no register is held across the loop for it);
    // only the sample's last, partial block needs per-lane clamping (to its last node).  A wave issues about
    // one instruction of any kind per five cycles, so what counts here is the number of instructions per copy:
    // the forms used in the step loop (issue_*_unrolled) are straight-line code with the LDS destinations as
    // constants and the block bases advanced by scalar adds.
    const int nfull = min(nblk, Lb / kBlk - jb0);   // owned blocks that are complete (all but possibly the last)
    const long long m_step = (long long)(dir ? -kBlk : kBlk) * ms2 * (long long)sizeof(TM);   // from one block's base to the next
    const long long m_first = (long long)(dir ? Lb - kBlk - jb0 * kBlk : jb0 * kBlk) * ms2 * (long long)sizeof(TM);
    const long long h_step = (long long)(dir ? -kBlk : kBlk) * 4;
    const long long h_first = (long long)(dir ? Lb - kBlk - flo * kBlk : flo * kBlk) * 4;
    const unsigned lds_base_u = opaque_uniform((int)lds_base);
    auto match_partial = [&](const int par, const int ob, const unsigned long long mrow) __attribute__((always_inline)) {
        const int pm = (jb0 + ob) * kBlk + lane, pmc = pm < Lb ? pm : Lb - 1;
        dma_elem_u<TM>(lds_base_u + (unsigned)stage_m_of(par, ob & (kTileWaves - 1), ob / kTileWaves) * 4u, mrow,
                       (unsigned)((dir ? Lb - 1 - pmc : pmc) * ms2) * (unsigned)sizeof(TM));
    };
    auto issue_match_unrolled = [&](auto parity, const int s2) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parity)::value;
        const int row = dir ? Tb - 1 - s2 : s2;
        const unsigned long long mrow = uniform_address(match_c + (unsigned)(row * ms1) * (unsigned)sizeof(TM));
        const unsigned lane_off = (unsigned)((dir ? kBlk - 1 - lane : lane) * ms2) * (unsigned)sizeof(TM);
        unsigned long long base = mrow + (unsigned long long)m_first;
#pragma unroll
        for (int ob = 0; ob < kPartBlocks; ++ob) {
            if (ob >= nfull) break;
            dma_elem_u<TM>(lds_base_u + (unsigned)stage_m_of(PAR, ob & (kTileWaves - 1), ob / kTileWaves) * 4u, base, lane_off);
            base += (unsigned long long)m_step;
        }
        if (nfull < nblk) match_partial(PAR, nfull, mrow);
    };
    auto issue_rows = [&](const int s2) __attribute__((always_inline)) {    // table rows of the foreign blocks (all complete) for step s2
        const int row = dir ? Tb - 1 - s2 : s2, par = s2 & 1;
        unsigned long long base = uniform_address(hat_c + (unsigned)(row * L) * 4u) + (unsigned long long)h_first;
        const unsigned lane_off = (unsigned)(dir ? kBlk - 1 - lane : lane) * 4u;
        for (int q = 0; q < jb0 - flo; ++q, base += (unsigned long long)h_step)
            dma_dword_agent_u(lds_base_u + (unsigned)stage_f_of(par, kTileWaves - 1 - (q & (kTileWaves - 1)), q / kTileWaves) * 4u, base, lane_off);
        dma_dword_agent_u(lds_base_u + (unsigned)stage_o(par) * 4u, uniform_address(off_c + (unsigned)(row * NBK) * 8u),
                          (unsigned)(lane < 2 * NBK ? lane : 2 * NBK - 1) * 4u);
        rows_issued = s2;
    };
    // called in phase A of step s: make sure what phase B of step s reads has landed, request step s + 1
    auto fetch_step = [&](auto parity_next, const int s) __attribute__((always_inline)) {
        // parity_next: the buffers of step s + 1 (those of step s have the other parity)
        constexpr int PN = decltype(parity_next)::value;
        wait_vmem_all();   // everything requested a step ago
        const bool need_rows = consumer && s < Tb - 1;
        if (need_rows) {
            snapshot = __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, lds_raw[stage_p(s & 1)]));   // requested a step ago
            if (snapshot > seen) seen = snapshot;
            if (rows_issued < s) {   // not requested yet: the producer is less than two steps ahead, poll its word
                int spins = 0;
                while (seen < s) {   // the rows of step s are published once the word reaches s
                    seen = __builtin_amdgcn_readfirstlane(load_agent(below));
                    if (seen >= s) break;
                    __builtin_amdgcn_s_sleep(2);
                    if (++spins > kSpinLimit) { s_abort = 1; break; }
                }
                if (seen >= s) { issue_rows(s); wait_vmem_all(); }
            }
        }
        if (s + 1 < Tb) {
            if (!consumer) issue_match_unrolled(parity_next, s + 1);   // (a consumer group's waves request their own rows)
            if (consumer && s + 1 < Tb - 1) {
                // The waves of a consumer group each request the table row of their own foreign block for step
                // s + 1 (own_requests), all on the same evidence: the snapshot of the producer's progress word that
                // was requested a step ago (every copy of a step has landed before the step's last barrier: the
                // fetcher, too, waits for its requests at the top of phase B).  Here only what the waves share: the
                // offsets of that row, and the next snapshot.
                if (snapshot >= s + 1) {
                    const int row = dir ? Tb - 2 - s : s + 1;
                    dma_dword_agent_u(lds_base_u + (unsigned)stage_o(PN) * 4u, uniform_address(off_c + (unsigned)(row * NBK) * 8u),
                                      (unsigned)(lane < 2 * NBK ? lane : 2 * NBK - 1) * 4u);
                    rows_issued = s + 1;
                }
                dma_dword_agent(lds_base_u + (unsigned)stage_p(PN) * 4u, below, 0u);
            }
        }
    };
    // Every wave of a consumer group, in phase A of step s: request what its own phase B of step s + 1 reads -- the
    // match row of the block(s) it owns and, once the fetcher's published progress covers step s + 1, the table
    // row of its foreign block(s).  One or two copies per wave instead of all of them queued behind each other in
    // the fetcher, whose arrival at the barrier was what the group's tile waves waited for.  A wave consumes only
    // what it requested itself, after waits of its own (top of phase B; the fetcher at the top of its fetch).
    auto own_requests = [&](auto parity_next, const int s) __attribute__((always_inline)) {
        constexpr int PN = decltype(parity_next)::value;
        if (s + 1 >= Tb) return;
        const int row = dir ? Tb - 2 - s : s + 1;
        if (owner) {
            const unsigned long long mrow = uniform_address(match_c + (unsigned)(row * ms1) * (unsigned)sizeof(TM));
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                if (u == 1 && wave + kTileWaves >= nblk) break;
                const int pm = p_own + u * kTileWaves * kBlk, pmc = pm < Lb ? pm : Lb - 1;
                dma_elem_u<TM>(lds_base_u + (unsigned)stage_m(PN, u) * 4u, mrow,
                               (unsigned)((dir ? Lb - 1 - pmc : pmc) * ms2) * (unsigned)sizeof(TM));
            }
        }
        if (s + 1 < Tb - 1 && f_blk[0] >= 0) {
            const int known = __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, lds_raw[stage_p(PN ^ 1)]));
            if (known >= s + 1) {
                const unsigned long long hrow = uniform_address(hat_c + (unsigned)(row * L) * 4u);
                int ln = lane;   // (redone every step: ahead of the loop it would hold a register per slot)
                asm volatile("" : "+v"(ln));
#pragma unroll
                for (int u = 0; u < kFetchSlots; ++u) {
                    if (f_blk[u] < 0) break;
                    const int pf = f_blk[u] * kBlk + ln;   // foreign blocks are complete
                    dma_dword_agent_u(lds_base_u + (unsigned)stage_f(PN, u) * 4u, hrow, (unsigned)(dir ? Lb - 1 - pf : pf) * 4u);
                }
            }
        }
    };
    auto uniform_double = [&](double v) -> double {
        const long long bits = __builtin_bit_cast(long long, v);
        const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(bits & 0xffffffffLL));
        const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(bits >> 32));
        return __builtin_bit_cast(double, ((long long)hi << 32) | (long long)lo);
    };
    if (fetcher && Tb > 1) {   // what phase B of step 1 needs
        issue_match_unrolled(std::integral_constant<int, 1>{}, 1);
        if (consumer && 1 < Tb - 1) dma_dword_agent(lds_base + (unsigned)stage_p(1) * 4u, below, 0u);
    }
    wait_vmem_all();
    __syncthreads();

    bool aborted = false;
    // The read-out needs what the lane of position L_b-1 computed in the last step, and that step's reference.  The
    // last step leaves them in LDS: as variables they would hold three registers across the whole loop.
    VT *const last_v = reinterpret_cast<VT *>(lds_raw + kLdsLastV) + wave * kBlk + lane;
    *last_v = (VT)DAGX_NEG_INF;
    // One step; CUR = parity of the buffers that hold step s-1 (compile-time: immediate LDS offsets).
    // UNL: every lower block is a predecessor block (compile-time: the hot path has no branch on it).
    auto step = [&](auto parity, auto unl, const int s) __attribute__((always_inline)) {
        constexpr int CUR = decltype(parity)::value, NXT = CUR ^ 1;
        constexpr bool UNL = decltype(unl)::value;
        const int t = dir ? Tb - 1 - s : s;
        // ---------------- phase A: tile mat-vecs (LDS and registers only); the fetcher's copies ----------------
        if (__builtin_expect(fetcher, 0)) fetch_step(parity, s);   // step s + 1 uses the buffers that now hold step s - 1
        double rl64 = 0.0;
        float rl;
        if constexpr (WIDE) { rl64 = relb64[CUR * kMaxBlocksFast + (lane & 15)]; rl = (float)rl64; }
        else rl = lds_l15[kLdsRelb + CUR * kMaxBlocksFast];
        auto read_e = [&](const int sl, EV (&ev)[4]) __attribute__((always_inline)) {
            const EV *src = ev_l15 + opaque_uniform(e_off[sl]);
#pragma unroll
            for (int q = 0; q < 4; ++q) ev[q] = src[CUR * kEbufPar + 16 * q];
        };
        EV eva[4], evb[4];
        read_e(0, eva);
        if constexpr (!WIDE) read_e(1, evb);
        float tail[kTailRows > 0 ? kTailRows : 1];
        if constexpr (WIDE) {   // (requested now, used behind the first two tiles)
#pragma unroll
            for (int u = 0; u < kTailRows; ++u) tail[u] = tail_lane[u * kBlk];
        }
        // Rvec: lane Jb holds the scale of position block Jb = max offset over its predecessor blocks
        const float rpre = row16_prefix_max(rl);
        const float dmax = lane_bcast(rpre, 15);
        const float d_s = dmax > DAGX_NEG_INF ? dmax : 0.f;  // next step's reference = cref + d_s
        auto block_scale = [&](int Jb) -> float {
            if constexpr (UNL) return lane_bcast(rpre, Jb);
            else return lane_bcast(row16_max(((lane & 15) >= tile_ilo(Jb, W) && (lane & 15) <= Jb) ? rl : DAGX_NEG_INF), 0);
        };
        auto tile_step = [&](const int sl, const Tile &tile, const EV (&ev)[4]) __attribute__((always_inline)) {
            // the raw product (at most 64 * 2^112): the factor exp(off_I - R_J) that brings the tiles of one
            // output block to a common scale is applied by the block's owner, for all its tiles at once
            EV acc = 0;
            if (__builtin_expect(s >= s_lo[sl] && s <= s_hi[sl], 1)) acc = tile_dot(tile, ev[0], ev[1], ev[2], ev[3]);
            ev_lane[opaque_uniform(part_off[sl])] = acc;
        };
        // (here, with the reads of this step's vectors in flight: its one LDS read then costs no wait of its own)
        if (consumer) own_requests(parity, s);
        tile_step(0, t0, eva);
        if constexpr (WIDE) {   // one set of float64 e values at a time: a second set does not fit the register file
            read_e(1, eva);
            tile_step(1, t1, eva);
            read_e(2, eva);
            EV acc = 0;
            if (__builtin_expect(s >= s_lo[2] && s <= s_hi[2], 1)) acc = tile_dot_tail(t2, tail, eva[0], eva[1], eva[2], eva[3]);
            ev_lane[opaque_uniform(part_off[2])] = acc;
        } else {
            read_e(2, eva);
            tile_step(1, t1, evb);
            tile_step(2, t2, eva);
        }
        __syncthreads();
        // ---------------- phase B ----------------
        // Every earlier store of this wave is complete (those of step s-1 were issued a whole step ago, so
        // this costs nothing), which lets the progress word below run one step behind instead of two.
        // The copies this wave requested in phase A (for step s + 1) have landed, too -- they were issued one
        // to two thousand cycles ago -- so that after the barrier that ends this step every wave may read any of
        // them (the progress snapshot the whole group decides on).
        wait_vmem_all();
        // (set in phase A only, by the fetcher; requested here with the other LDS reads, looked at behind the barrier)
        const int gave_up_v = consumer ? s_abort : 0;
        const double cnext = cref + (double)d_s;
        // (1) hand-over: rows of step s from the producer groups -> ebuf/relb of the next step
        if (consumer && s < Tb - 1) {
#pragma unroll
            for (int u = 0; u < kFetchSlots; ++u) {
                if (f_blk[u] < 0) continue;
                const int I = f_blk[u];
                const float fh = lds_lane[stage_f(NXT, u)];
                EV ef = LN::exp2s(fh * kLog2e);
                ef = (fh > -3.0e38f && ef < tiny_up) ? tiny_up : ef;   // (as in own_block)
                ev_lane[kEvEbuf + NXT * kEbufPar + I * kBlk] = I * kBlk + lane < Lb ? ef : (EV)0;
                const double o = reinterpret_cast<const double *>(lds_raw + stage_o(NXT))[I];
                if (lane == 0) {
                    if constexpr (WIDE) relb64[NXT * kMaxBlocksFast + I] = o > (double)DAGX_NEG_INF ? o - cnext : (double)DAGX_NEG_INF;
                    else relb[NXT * kMaxBlocksFast + I] = o > (double)DAGX_NEG_INF ? (float)(o - cnext) : DAGX_NEG_INF;
                }
            }
        }
        // (2) sum the tiles of each owned block
        auto own_block = [&](const int Jb, const int poff, const int nt, const int p, const int node,
                             const float mv) __attribute__((always_inline)) -> VT {
            // partial sums (rows past the last tile are never written and hold 0), each times the factor that
            // brings its tile to the block's scale: lane I of every 16-lane row of `fac` holds exp(off_I - R) for
            // predecessor block I, capped at 1 -- a predecessor's factor never exceeds it, and the lanes of blocks
            // that are no predecessors (whose rows hold 0) must not turn into inf * 0 -- and 0 for a dead block
            // whose successors are alive.
            // (Computed here, behind the barrier, from a copy of the offsets the compiler cannot trace back into
            //  phase A: hoisted in front of the tiles this arithmetic lengthened every wave's phase A.)
            const EV *prd = ev_lane + opaque_uniform(poff);
            // the first eight partial sums are requested before anything else, all at once: one LDS round trip
            // for them (read four at a time, next to their use, they cost two, one behind the other)
            EV pr[8];
#pragma unroll
            for (int u = 0; u < (WIDE ? 4 : 8); ++u) pr[u] = prd[u * kBlk];   // (float64 sums: four at a time, for want of registers)
            asm volatile("" ::: "memory");
            float rlb = rl;
            asm volatile("" : "+v"(rlb));
            const float R = block_scale(Jb);
            // exp2(clamp(x, floor, 0)), floor = -inf (lower sweep) or -126 (upper sweep: a live block's factor never
            // flushes; a dead block's rows hold 0 whatever stands in front of them).  -inf - R gives the floor;
            // finite - -inf (+inf) gives 0, factor 1, and -inf - -inf (NaN) the floor (the median of three with a NaN
            // among them is the smallest of the others), both in front of rows that hold 0.
            EV fac;
            if constexpr (WIDE) {   // (the offsets' difference in float64: see Lin<true>::exp2_with)
                double rlb64 = rl64;
                asm volatile("" : "+v"(rlb64));
                // (R is the float32 rounding of the largest offset, so the block that sets the scale may lie a rounding
                //  error above it: capped at 2, not at 1, or it would lose that sliver of its mass in every step)
                const double x = (rlb64 - (double)R) * (double)kLog2e;
                fac = LN::exp2_with(__builtin_fmax(__builtin_fmin(x, 1.0), (double)fac_floor), 0);
            } else {
                fac = LN::exp2u(__builtin_amdgcn_fmed3f((rlb - R) * kLog2e, fac_floor, 0.f));
            }
            // partial row u belongs to predecessor block ilo + u (ilo = 0 when every lower block is a predecessor):
            // with the factors shifted down by ilo lanes, row u takes its factor from lane u by DPP broadcast
            EV facu = fac;
            if constexpr (!UNL) {
                const int from = ((lane & 15) + tile_ilo(Jb, W)) << 2;
                if constexpr (WIDE) {
                    const long long bits = __builtin_bit_cast(long long, fac);
                    const unsigned lo = (unsigned)__builtin_amdgcn_ds_bpermute(from, (int)(bits & 0xffffffffLL));
                    const unsigned hi = (unsigned)__builtin_amdgcn_ds_bpermute(from, (int)(bits >> 32));
                    facu = __builtin_bit_cast(double, ((long long)hi << 32) | (long long)lo);
                } else {
                    facu = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from, __builtin_bit_cast(int, fac)));
                }
            }
            EV tot;
            scaled_sum4<0>(tot, facu, pr[0], pr[1], pr[2], pr[3]);
            if constexpr (WIDE) {
#pragma unroll
                for (int u = 0; u < 4; ++u) pr[u] = prd[(4 + u) * kBlk];
                scaled_sum4<4>(tot, facu, pr[0], pr[1], pr[2], pr[3]);
            } else {
                scaled_sum4<4>(tot, facu, pr[4], pr[5], pr[6], pr[7]);
            }
            if (__builtin_expect(nt > 8, 0)) {
                scaled_sum4<8>(tot, facu, prd[8 * kBlk], prd[9 * kBlk], prd[10 * kBlk], prd[11 * kBlk]);
                scaled_sum4<12>(tot, facu, prd[12 * kBlk], prd[13 * kBlk], prd[14 * kBlk], prd[15 * kBlk]);
            }
            // upper sweep: more than every product that may have been flushed on the way to this sum (64 per tile
            // under 2^-126 each, 16 tiles, 16 scaled partial sums under 2^-126)
            tot += flush_up;
            // Dead cells come out as -inf by arithmetic alone (every test here is an instruction of the busiest
            // SIMD): no live predecessor gives tot = 0 and log2 = -inf (R is then finite or -inf, never +inf), a
            // match of -inf adds -inf; only the band has to be imposed.  A block without any live cell has
            // vmax = -inf: its offset (finite reference + -inf) and relative offset are -inf, and its residuals
            // are taken against -3e38 instead, which leaves them -inf and their exponentials 0.
            const bool inband = p >= s && p <= slack + s;
            VT vt;
            if constexpr (WIDE) vt = inband ? ((double)R + LN::log2u_wide(tot) * 0.6931471805599453) + (double)mv : (double)DAGX_NEG_INF;
            else vt = inband ? (R + LN::log2u(tot) * kLn2) + mv : DAGX_NEG_INF;
            const float v = (float)vt;
            const float vmax = wave64_max(v);
            const double offn = cref + (double)vmax;
            float fh;   // the residual against the block's maximum (formed from the float64 value in the wide variant)
            if constexpr (WIDE) fh = (float)(vt - (double)fmaxf(vmax, -3.0e38f));
            else fh = v - fmaxf(vmax, -3.0e38f);
            EV e;
            if constexpr (WIDE) {
                // exp(v - vmax) not from the rounded v but from the sum itself: tot * exp(R + match - vmax) in float64
                // (the shift of the staged transitions taken out, that of the float64 numbers staying in), so that a
                // cell hundreds of nats under its reference hands on what it received to float64 accuracy
                const double x = ((((double)R - (double)vmax) + (double)mv) * (double)kLog2e) - (double)kShiftLinksWide;
                // (a block without a live cell has vmax = -inf and exponentials 0 -- unless its sums are NaNs, which the
                //  maximum skipped and which must stay NaNs)
                e = !inband ? 0.0 : (vmax > -3.0e38f ? LN::times_exp2(tot, x) : (tot == tot ? 0.0 : tot));
            } else {
                e = LN::exp2s(fh * kLog2e);
            }
            e = (fh > -3.0e38f && e < tiny_up) ? tiny_up : e;   // upper sweep: a live cell never flushes (a NaN stays one)
            ev_lane[opaque_uniform(kEvEbuf + NXT * kEbufPar + Jb * kBlk)] = e;
            if (lane == 0) {
                if constexpr (WIDE) relb64[NXT * kMaxBlocksFast + Jb] = (double)vmax - (double)d_s;
                else relb[NXT * kMaxBlocksFast + Jb] = vmax - d_s;
                store_agent(off_at(t, Jb), offn);
            }
            if (p < Lb) store_agent(hat_at(t, node), fh);
            return vt;   // relative to cref; the last step's value at position L_b-1 is the read-out
        };
        const bool last_step = s == Tb - 1;
        if (owner) {
            const VT v1 = own_block(Jown, own_part_off, nt_own, p_own, node_own, dma_decode<TM>(__builtin_bit_cast(unsigned, lds_lane[stage_m(NXT, 0)])));
            if (last_step) {
                *last_v = v1;
                if (lane == 0) reinterpret_cast<double *>(lds_raw + kLdsLastC)[wave] = cref;
            }
        }
        if (wave + kTileWaves < nblk) {   // a second owned block (many narrow blocks)
            const int Jb = Jown + kTileWaves, p = p_own + kTileWaves * kBlk, node = dir ? Lb - 1 - p : p;
            const VT v2 = own_block(Jb, own_part_off + kTileWaves * kPartRows * kBlk, Jb - tile_ilo(Jb, W) + 1, p, node,
                                       dma_decode<TM>(__builtin_bit_cast(unsigned, lds_lane[stage_m(NXT, 1)])));
            if (last_step && p == Lb - 1) *last_v = v2;   // the lane of position L_b-1 keeps that block's value
        }
        __syncthreads();
        if (__builtin_amdgcn_readfirstlane(gave_up_v)) {   // only a consumer's own spin can set the flag; dealt with behind the loop
            aborted = true;
            return;
        }
        // Every wave has seen its stores of step s-1 complete (the wait at the top of phase B).
        if (__builtin_expect(tid == 0 && producer && s >= 1, 0)) store_agent(prog + g, s - 1);
        cref = uniform_double(cnext);
    };

    auto sweep = [&](auto unl) __attribute__((always_inline)) {
        for (int s = 1; s < Tb; s += 2) {
            step(std::integral_constant<int, 0>{}, unl, s);
            if (aborted) return;
            if (s + 1 < Tb) {
                step(std::integral_constant<int, 1>{}, unl, s + 1);
                if (aborted) return;
            }
        }
    };
    if (unlimited) sweep(std::true_type{}); else sweep(std::false_type{});
    if (aborted) {
        // a producer never showed up: hand the sample to the exact kernel and let consumers go on
        if (tid == 0) {
            store_agent(risk, 1);
            store_agent(prog + g, 1 << 30);
        }
        return;
    }
    // read-out: the value of position L_b-1 after the last step (T_b = 1 was written above)
    if (Tb > 1) {
        const int pl = Lb - 1, Jl = pl / kBlk;
        if (Jl >= jb0 && Jl < jb1 && ((Jl - jb0) & (kTileWaves - 1)) == wave && (pl & (kBlk - 1)) == lane) {
            const VT v_last = *last_v;   // (written by this very lane)
            const double cref_last = reinterpret_cast<const double *>(lds_raw + kLdsLastC)[wave];   // (by lane 0 of this wave)
            const double z = v_last > (VT)DAGX_NEG_INF ? cref_last + (double)v_last : (double)DAGX_NEG_INF;
            a.logz[slot * a.B + b] = z; if (slot == a.loss_dir) a.loss[b] = (float)z; store_agent(a.zfast + slot * a.B + b, z);
        }
    }
    if (producer) {
        wait_vmem_all();
        __syncthreads();
        if (tid == 0) store_agent(prog + g, Tb - 1);
    }
}

// The two read-outs of a sample's tile sweeps bracket log Z: one sweep rounds everything the linear domain
// cannot hold down to 0, the other up to the smallest number it holds.  Where they agree, what was flushed carried
// no mass that matters and either read-out is log Z to the tolerance; where they do not (or one is not finite,
// or a NaN) the sample is done again: by the wide sweeps, then by the log-domain kernel.  The tolerance bounds the
// mass the upper sweep has rounded up, which the gradients would see as posteriors of that size where the true ones
// are 0: 5e-5, half of what the gradients are held to.  On top of it comes what rounding alone leaves between two
// sweeps.  The float32 sweeps carry cell values as float32 numbers relative to a float64 reference: measured between
// an alpha and a beta sweep up to 1.5e-5 at |log Z| = 800 on benign inputs and 3e-5 ... 5e-5 at 2600 ... 3500, hence
// the term 1e-7 |Z|; but never more than 1e-4, what the gradients are held to, however large |log Z| (the few
// samples of long, peaked graphs whose read-outs differ by more through rounding alone cost a pass of the wide
// sweeps).  The wide sweeps carry them as float64 numbers whose
// logarithm comes from v_log_f32 of a fraction in [1/2, 1), 1e-7 absolute per step: 1e-8 |Z| covers it.  (With
// float32 cell values the wide sweeps needed 2e-4 + 2e-7 |Z|, and that passed upper sweeps that had rounded
// 3e-4 ... 6e-4 of mass up: their transitions are clamped at exp(-175) times the scale, which is not nothing when
// the path that carries the mass lies as deep.)
__device__ __forceinline__ bool readouts_disagree(double za, double zb, bool wide) {
    if (!(za > (double)DAGX_NEG_INF) || !(zb > (double)DAGX_NEG_INF) || za != za || zb != zb) return true;
    return fabs(za - zb) > (wide ? 1e-8 * fabs(zb) + 5e-5 : fmin(1e-7 * fabs(zb) + 5e-5, 1e-4));
}

template <typename TM, typename TL, bool WIDE>
__global__ __launch_bounds__(kTileWaves * kWave) void dag_sweep_tiles_kernel(SweepArgs a) {
    extern __shared__ float lds_raw[];
    __shared__ int gstart[kTileCap + 2];
    __shared__ int s_ticket, s_abort;
    const int tid = threadIdx.x;
    const int C = a.C;
    // The wide launch behind a float32 launch that flagged nothing (the usual case) ends here, after one load: the
    // float32 launch counts the samples it flags in word 2 of the pipeline words, the wide launch clears it.
    if constexpr (WIDE) { if (a.sync[2] == 0) return; }
    if (tid == 0) { s_ticket = atomicAdd(a.sync, 1); s_abort = 0; }
    __syncthreads();
    // ticket -> (group, sweep, sample): first group 0 of every sweep of every sample, then every group 1, and so on.
    // Every group waits only on groups with a smaller ticket, so a waiting workgroup's producers have already
    // started; and the workgroups that the dispatcher reaches last (it needs several microseconds for the grid)
    // are consumers, which could not start any sooner than their producers' first rows anyway.  The two sweeps of a
    // sample are 8 tickets apart, the workgroups of a sample a multiple of 8: they share an XCD and its L2.
    const int k = __builtin_amdgcn_readfirstlane(s_ticket);
    const int B8 = (a.B + 7) & ~7;
    const int runs = a.ndir * (B8 / 8);   // runs of eight (sweep, sample) pairs
    const int g = k / (8 * runs), run = (k / 8) % runs;
    const int b_k = (run / a.ndir) * 8 + (k % 8);
    const bool has_sample = g < C && b_k < a.B;
    const int b = has_sample ? b_k : 0, slot = has_sample ? run % a.ndir : 0;
    // a launch for flagged samples only (the wide variant behind the float32 one): the workgroups of the others
    // leave at once, through the same bookkeeping
    const bool skip = has_sample && a.only_flagged && a.flags[b] != 1;
    if (has_sample && !skip) sweep_tiles_group<TM, TL, WIDE>(a, b, slot, g, lds_raw, gstart, &s_abort);
    // ---- leaving ----
    wait_vmem_all();   // this wave's stores (table rows, read-outs) are complete
    __syncthreads();
    if (tid == 0) {
        if (has_sample) {
            int *left = a.sync + 16 + a.ndir * a.B * C + b, *risk = left + a.B;
            const int n = __hip_atomic_fetch_add(left, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
            if (n == a.ndir * C) {   // every workgroup of the sample has left
                bool bad = load_agent(risk) != 0;
                const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
                if (!bad && lengths_ok(Lb, Tb, a.L, a.T)) {
                    bad = readouts_disagree(load_agent(a.zfast + b), load_agent(a.zfast + a.B + b), WIDE);
                }
                if (!skip) a.flags[b] = bad ? 1 : (WIDE ? 2 : 0);   // 1: still to be done; 2: settled by the wide variant
                if (!WIDE && bad) __hip_atomic_fetch_add(a.sync + 2, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                for (int d = 0; d < a.ndir; ++d)
                    for (int q = 0; q < C; ++q) store_agent(a.sync + 16 + (d * a.B + b) * C + q, 0);
                store_agent(left, 0);
                store_agent(risk, 0);
                for (int d = 0; d < a.ndir; ++d) store_agent(a.zfast + d * a.B + b, 0.0);
            }
        }
        const int n_all = __hip_atomic_fetch_add(a.sync + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
        if (n_all == (int)gridDim.x) { store_agent(a.sync, 0); store_agent(a.sync + 1, 0); if (WIDE) store_agent(a.sync + 2, 0); }
    }
}

// In front of a forward that starts with the float64 sweeps: every sample marked "still to be done", and the count the
// float32 launch would have left, so that the float64 launch does not take itself for idle.
__global__ void dag_mark_all_kernel(int *flags, int B, int *sync) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < B) flags[i] = 1;
    if (i == 0) store_agent(sync + 2, B);
}

__global__ void dag_fill_int_kernel(int *p, int n, int v) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// ================================================================================================
// Gradients
// ================================================================================================

__device__ __forceinline__ bool finite_d(double z) { return z > (double)DAGX_NEG_INF && z < (double)__builtin_huge_valf(); }

// Clearing the part of grad_links that the tile kernel does not write.  Per sample:
//   - valid lengths, T_b >= 2, finite Z: the tile kernel writes the entries with i + d + 1 < L_b, so row i
//     is cleared from d = max(0, L_b - 1 - i) on;
//   - otherwise the gradient is zero everywhere and the whole sample is cleared.
// A workgroup of four waves owns `rows` consecutive rows of one sample, a wave clears a row at a time:
// 16-byte stores between element-wise head and tail (row starts are only element-aligned).
typedef uint32_t fill_u32x4 __attribute__((ext_vector_type(4)));
struct ZeroJob {
    unsigned char *base; int elem;       // grad_links and its element size (2 or 4)
    const int64_t *out_len, *tgt_len; const double *logz;   // logz: [2][B], the second row is Z
    int B, T, L, translen;
    int rows, chunks;                    // rows per workgroup, workgroups per sample
    int blocks;                          // B * chunks; 0: nothing to clear
};
__device__ __forceinline__ void zero_elem(unsigned char *p, int elem) {
    if (elem == 4) *reinterpret_cast<uint32_t *>(p) = 0u; else *reinterpret_cast<uint16_t *>(p) = 0;
}
__device__ __forceinline__ void zero_part(const ZeroJob &z, int block) {
    const int tid = threadIdx.x;
    const int b = block / z.chunks, chunk = block % z.chunks;
    const int Lb = (int)z.out_len[b], Tb = (int)z.tgt_len[b];
    const double Z = z.logz[z.B + b];
    const bool tiled = lengths_ok(Lb, Tb, z.L, z.T) && Tb >= 2 && finite_d(Z);
    const int i_end = (chunk + 1) * z.rows < z.L ? (chunk + 1) * z.rows : z.L;
    const int lane = tid & (kWave - 1);
    for (int i = chunk * z.rows + (tid >> 6); i < i_end; i += (int)(blockDim.x >> 6)) {   // one wave per row
        int d0 = tiled ? Lb - 1 - i : 0;
        if (d0 < 0) d0 = 0;
        if (d0 >= z.translen) continue;
        unsigned char *row = z.base + ((int64_t)b * z.L + i) * z.translen * z.elem;
        const unsigned misalign = (unsigned)(reinterpret_cast<uintptr_t>(row) & 15u);
        const unsigned s = (unsigned)(d0 * z.elem), e = (unsigned)(z.translen * z.elem);   // byte range [s, e) of the row
        unsigned body = ((s + misalign + 15u) & ~15u) - misalign; if (body > e) body = e;  // first 16-byte boundary at or after s
        const unsigned body_end = body + ((e - body) & ~15u);
        for (unsigned o = s + lane * z.elem; o < body; o += kWave * z.elem) zero_elem(row + o, z.elem);
        for (unsigned o = body + lane * 16u; o < body_end; o += kWave * 16u) *reinterpret_cast<fill_u32x4 *>(row + o) = fill_u32x4{0u, 0u, 0u, 0u};
        for (unsigned o = body_end + lane * z.elem; o < e; o += kWave * z.elem) zero_elem(row + o, z.elem);
    }
}

// grad_match[b][t][j] = g_b * exp(alpha + beta - match - Z), Z = beta read-out; 0 outside the sample,
// where match is +-inf, or when Z is not finite.  The first zero.blocks workgroups of the launch clear
// the grad_links buffer instead (one launch less in front of the tile kernel).
template <typename TM>
__device__ __forceinline__ void grad_match_cell(
    const float *__restrict__ grad_out, int64_t gstride, const float *__restrict__ ahat, const float *__restrict__ bhat,
    const double *__restrict__ aoff, const double *__restrict__ boff, const double *__restrict__ logz,
    const TM *__restrict__ match, int64_t ms0, int64_t ms1, int64_t ms2,
    const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len, int B, int T, int L, int NBK,
    TM *__restrict__ grad_match, int b, int t, int j) {
    if (j >= L) return;
    const int Lb = (int)out_len[b], Tb = (int)tgt_len[b];
    const int64_t o = ((int64_t)b * T + t) * L + j;
    float r = 0.f;
    if (lengths_ok(Lb, Tb, L, T) && t < Tb && j < Lb) {
        const double Z = logz[B + b];
        const float m = to_float(match[b * ms0 + t * ms1 + j * ms2]);
        if (finite_d(Z) && m > DAGX_NEG_INF && m < __builtin_huge_valf()) {
            const int64_t ob = ((int64_t)b * T + t) * NBK;
            const double k = aoff[ob + j / kBlk] + boff[ob + (Lb - 1 - j) / kBlk] - Z;  // -inf if a block is dead
            // (summed in float64: with token log-probabilities a hundred nats apart the four terms are hundreds each and
            //  cancel, and float32 sums of them are off by 1e-4 of a posterior near 1)
            const float x = (float)((((double)ahat[o] + (double)bhat[o]) + k) - (double)m);
            r = grad_out[b * gstride] * fast_exp2(x * kLog2e);
        }
    }
    grad_match[o] = from_float<TM>(r);
}
template <typename TM>
__global__ __launch_bounds__(256) void dag_grad_match_kernel(
    const float *__restrict__ grad_out, int64_t gstride, const float *__restrict__ ahat, const float *__restrict__ bhat,
    const double *__restrict__ aoff, const double *__restrict__ boff, const double *__restrict__ logz,
    const TM *__restrict__ match, int64_t ms0, int64_t ms1, int64_t ms2,
    const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len, int B, int T, int L, int NBK,
    TM *__restrict__ grad_match, ZeroJob zero) {
    if ((int)blockIdx.x < zero.blocks) { zero_part(zero, blockIdx.x); return; }
    const int id = blockIdx.x - zero.blocks, nx = (L + 255) / 256;
    grad_match_cell<TM>(grad_out, gstride, ahat, bhat, aoff, boff, logz, match, ms0, ms1, ms2, out_len, tgt_len, B, T, L, NBK,
                        grad_match, id / (nx * T), (id / nx) % T, (id % nx) * 256 + (int)threadIdx.x);
}

// grad_links[b][i][d] = g_b * sum_{t=0}^{T_b-2} exp(alpha[t][i] + E[i][d] + beta[t+1][i+d+1] - Z), direct form
// (each term <= 1), for graphs the tile kernel does not take (L > 1024) and for the log-domain-only mode.
// Tile: RI rows x 64 transitions per workgroup.  The steps are walked in chunks of kDirectSteps: per chunk
// the alpha residuals of the rows (float32) and, per column, the beta residual plus every block offset of the
// step minus Z (float64: the offsets are large and cancel) are staged in LDS; a term is
// exp(float32(float64 sum) + E).
constexpr int kDirectSteps = 32;
template <typename TL, int RI>
__global__ __launch_bounds__(256) void dag_grad_links_kernel(
    const float *__restrict__ grad_out, int64_t gstride, const float *__restrict__ ahat, const float *__restrict__ bhat,
    const double *__restrict__ aoff, const double *__restrict__ boff, const double *__restrict__ logz,
    const TL *__restrict__ links, const int64_t *__restrict__ out_len, const int64_t *__restrict__ tgt_len,
    int B, int T, int L, int translen, int NBK, TL *__restrict__ grad_links) {
    constexpr int JW = 64 + RI;          // columns of beta touched by the tile (j = i+d+1)
    __shared__ float a_s[kDirectSteps][RI];     // alpha_hat[t][i]
    __shared__ double b_s[kDirectSteps][JW];    // beta_hat[t+1][j] + beta_off[t+1][blk(j)] + alpha_off[t][blk(i0)] - Z
    const int b = blockIdx.z;
    const int d0 = blockIdx.x * 64;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int Lb = (int)out_len[b], Tb = (int)tgt_len[b];
    TL *gl = grad_links + (int64_t)b * L * translen;
    const int d = d0 + lane;
    const bool ok = lengths_ok(Lb, Tb, L, T);
    const double Z = ok ? logz[B + b] : (double)DAGX_NEG_INF;
    const float g = grad_out[b * gstride];
    const float *al = ahat + (int64_t)b * T * L, *be = bhat + (int64_t)b * T * L;
    const double *ao = aoff + (int64_t)b * T * NBK, *bo = boff + (int64_t)b * T * NBK;
    // a workgroup walks the row tiles blockIdx.y, blockIdx.y + gridDim.y, ... of its column strip
    for (int i0 = blockIdx.y * RI; i0 < L; i0 += gridDim.y * RI) {
        const bool live = ok && finite_d(Z) && i0 < Lb - 1 && i0 + d0 + 1 < Lb && Tb >= 2;
        if (!live) {  // whole tile is zero
            for (int r = w; r < RI; r += 4) {
                const int i = i0 + r;
                if (i < L && d < translen) gl[(int64_t)i * translen + d] = from_float<TL>(0.f);
            }
            continue;
        }
        const int slack = Lb - Tb;
        const int jbase = i0 + d0 + 1;
        // useful steps for this tile: t in [tlo, thi]
        int tlo = jbase - 1 - slack; if (tlo < 0) tlo = 0;
        int thi = i0 + RI - 1; if (thi > Tb - 2) thi = Tb - 2;
        const int ablk0 = i0 / kBlk;         // RI divides 64: the rows of a tile share one alpha block
        float e[RI / 4], acc[RI / 4];
#pragma unroll
        for (int q = 0; q < RI / 4; ++q) {
            const int i = i0 + w + 4 * q, j = i + d + 1;
            acc[q] = 0.f;
            e[q] = (i < Lb - 1 && j < Lb && d < translen) ? to_float(links[((int64_t)b * L + i) * translen + d]) : DAGX_NEG_INF;
        }
        for (int c0 = tlo; c0 <= thi; c0 += kDirectSteps) {
            const int nt = thi - c0 + 1 < kDirectSteps ? thi - c0 + 1 : kDirectSteps;
            __syncthreads();   // the previous chunk's (or tile's) reads of the staged arrays are done
            for (int k = tid; k < nt * RI; k += 256) {
                const int t = c0 + k / RI, r = k % RI, i = i0 + r;
                a_s[k / RI][r] = i < Lb ? al[(int64_t)t * L + i] : DAGX_NEG_INF;
            }
            for (int k = tid; k < nt * JW; k += 256) {
                const int t = c0 + k / JW, c = k % JW, j = jbase + c;
                double v = (double)DAGX_NEG_INF;
                if (j < Lb) {
                    const double ka = ao[(int64_t)t * NBK + ablk0], kb = bo[(int64_t)(t + 1) * NBK + (Lb - 1 - j) / kBlk];
                    if (ka > (double)DAGX_NEG_INF && kb > (double)DAGX_NEG_INF)
                        v = (double)be[(int64_t)(t + 1) * L + j] + ((ka - Z) + kb);
                }
                b_s[k / JW][c] = v;
            }
            __syncthreads();
#pragma unroll
            for (int q = 0; q < RI / 4; ++q) {
                const int r = w + 4 * q;
                if (e[q] > DAGX_NEG_INF) {
                    const int c = r + lane;      // j - jbase
                    float sum = 0.f;
                    for (int k = 0; k < nt; ++k) {
                        const float x = (float)(b_s[k][c] + (double)a_s[k][r]) + e[q];
                        sum += fast_exp2(x * kLog2e);
                    }
                    acc[q] += sum;
                }
            }
        }
#pragma unroll
        for (int q = 0; q < RI / 4; ++q) {
            const int i = i0 + w + 4 * q;
            if (i < L && d < translen) gl[(int64_t)i * translen + d] = from_float<TL>(g * acc[q]);
        }
    }   // row tiles
}

// ------------------------------------------------------------------------------------------------
// grad_links, block-scaled form.  With ea = exp(alpha_hat), eb = exp(beta_hat) (both in [0,1]) and
// the per-step factor K_t = exp(alpha_off[t][blk(i)] + beta_off[t+1][blk(j)] - Z),
//     grad_links[i][j] = g * P[i][j] * sum_t (K_t^(1/2) ea[t][i]) * (K_t^(1/2) eb[t+1][j]),
// a matrix product over the steps, in fp32 on the matrix cores.  One wave per 32-row x 64-column
// tile: two 32x32 accumulator blocks, v_mfma_f32_32x32x2_f32 consuming two steps at a time.  Its
// operand layout (lane = 32 * k + row of A / column of B) is exactly what a coalesced load of two
// table rows gives, so the factors go from global memory through one exponential straight into the
// MFMA.  The per-step scale factors sit in a small LDS table, one read per operand and step pair.
//
// When the factored form is safe.  A term exp(alpha[t][i] + E + beta[t+1][j] - Z) is at most 1; its two
// factors are formed separately, and one of them can leave the float32 range although the term does not.
// With x_t = log K_t for the largest blocks of the tile, each factor carries half of it: a factor can only
// flush when its residual is below -87 - x_t / 2, and then every term it belongs to is below
// exp(x_t / 2 - 87) (the other residual and E are <= 0).  And a cell's sum over n steps is at most n exp(max x_t)
// (the residuals are <= 0), whatever its transition.  So the matrix product takes the steps with
// x_t <= 88 - log(n), n = the steps of the tile: their sums cannot leave float32 (its largest number is exp(88.7))
// and what the factored form loses of them is below exp(-43) per term.  The other steps of the tile (inputs whose
// posterior sits far under the block maxima: sharply peaked transitions, pinned nodes) are left out of the product
// (their scale entries are -inf) and added afterwards, by the same wave, in the direct form: every term from a
// float64 sum of its parts, the transition inside the exponent.  A sum that is not finite all the same (a NaN in
// the tables) sends the whole tile through the direct form.  All in the same launch, with no check afterwards and
// no second kernel.  (A looser bound for the product, 120, with a check of the sums and a second product under the
// tight bound where one overflowed, keeps moderately peaked inputs off the direct steps -- 0.036 against 0.048 ms
// for the x10 test batch -- but the second copy of the loop costs every tile 7 % through the register allocation.)
// ------------------------------------------------------------------------------------------------

typedef float f32x16 __attribute__((ext_vector_type(16)));
// log K_t up to which a step of a tile of n steps goes through the matrix product
__device__ __forceinline__ double safe_log_k(int n) { return (double)(88.0f - fast_log2((float)(n > 1 ? n : 1)) * kLn2); }

struct GradTileArgs {
    const float *grad_out; int64_t gstride;
    const float *ahat, *bhat; const double *aoff, *boff, *logz;
    const void *links; void *grad_links;
    const int64_t *out_len, *tgt_len;
    int B, T, L, translen, NBK;
    int ntile;                           // live (row block, column block) pairs of a full-length sample
    unsigned char tile_bi[kMaxBlocksFast * (kMaxBlocksFast + 1) / 2], tile_jt[kMaxBlocksFast * (kMaxBlocksFast + 1) / 2];
    // Work that rides in the same launch, behind the tile workgroups (which start first and are bound by
    // their chains of memory round trips, so that these streaming workgroups fill the machine around them):
    // the clearing of the part of grad_links no tile writes, and grad_match (four 64-cell pieces of a table
    // row per workgroup).  tile_blocks = 2 * ntile * B; then zero.blocks, then match_blocks.
    int tile_blocks, match_blocks;
    ZeroJob zero;
    const void *match; int match_dtype; int64_t ms0, ms1, ms2; void *grad_match;
};
// Four cells of grad_match per lane (one step t of one sample, 256 consecutive positions per wave): the same values
// as grad_match_cell, but every load is requested up front, without conditions (indices clamped into the tables; what
// must not count is masked at the end), so that a wave waits for two memory round trips (the sample's lengths, which
// the beta offsets' index needs, then everything else) instead of three per cell.  These workgroups ride in the
// slots the gradient tiles leave free, a few hundred at a time: what they cost is their latency.
template <typename TM>
__device__ __forceinline__ void grad_match_cells4(const GradTileArgs &a, const TM *__restrict__ match, TM *__restrict__ grad_match,
                                                   const int b, const int t, const int j0) {
    const int L = a.L, T = a.T, NBK = a.NBK;
    const int64_t row = ((int64_t)b * T + t) * L, ob = ((int64_t)b * T + t) * NBK;
    float m[4], ah[4], bh[4];
    double ao[4];
    int jc[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int j = j0 + u * kWave;
        jc[u] = j < L ? j : L - 1;
        m[u] = to_float(match[b * a.ms0 + t * a.ms1 + jc[u] * a.ms2]);
        ah[u] = a.ahat[row + jc[u]];
        bh[u] = a.bhat[row + jc[u]];
        ao[u] = a.aoff[ob + jc[u] / kBlk];
    }
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
    const double Z = a.logz[a.B + b];
    const float g = a.grad_out[b * a.gstride];
    const bool sample_ok = lengths_ok(Lb, Tb, L, T) && t < Tb && finite_d(Z);
    double bo[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        int q = (Lb - 1 - jc[u]) / kBlk;
        q = q < 0 ? 0 : (q < NBK ? q : NBK - 1);
        bo[u] = a.boff[ob + q];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int j = j0 + u * kWave;
        float r = 0.f;
        if (sample_ok && j < Lb && m[u] > DAGX_NEG_INF && m[u] < __builtin_huge_valf()) {
            const double k = ao[u] + bo[u] - Z;  // -inf if a block is dead
            const float x = (float)((((double)ah[u] + (double)bh[u]) + k) - (double)m[u]);   // (float64: see grad_match_cell)
            r = g * fast_exp2(x * kLog2e);
        }
        if (j < L) grad_match[row + j] = from_float<TM>(r);
    }
}

__device__ __forceinline__ void grad_side_jobs(const GradTileArgs &a, int id) {
    if (id < a.zero.blocks) { zero_part(a.zero, id); return; }
    id -= a.zero.blocks;
    const int nx = (a.L + 255) / 256;
    const int b = id / (nx * a.T), t = (id / nx) % a.T, j0 = (id % nx) * 256 + (int)threadIdx.x;
    switch (a.match_dtype) {
        case DAGX_F32: grad_match_cells4<float>(a, static_cast<const float *>(a.match), static_cast<float *>(a.grad_match), b, t, j0); break;
        case DAGX_F16: grad_match_cells4<__half>(a, static_cast<const __half *>(a.match), static_cast<__half *>(a.grad_match), b, t, j0); break;
        default: grad_match_cells4<bf16_t>(a, static_cast<const bf16_t *>(a.match), static_cast<bf16_t *>(a.grad_match), b, t, j0); break;
    }
}

// The direct form of one 32 x 64 tile, computed by one wave (see above for when).  Lane (half, l32)
// owns the columns j0 + l32 and j0 + 32 + l32 and the rows i0 + 8 q + 4 half + m (q, m < 4): cell (jh, v) of a
// lane is exp(float32(float64(beta side of its column) + float64(alpha residual of its row)) + E), summed over
// the steps; one column half after the other (16 accumulators and 16 link values live at a time).
// ONLY_OVER: only the steps whose log K_t exceeds safe_log_k (the matrix-core loop left exactly those out), added to
// what that loop found for the other steps (post[column half][v], the posterior sums of the lane's cells).
template <typename TL, bool ONLY_OVER>
__device__ __forceinline__ void grad_tile_direct(
    const float *al_f, const float *be_f, const double *ao, const double *bo, double Z, const TL *lk, TL *gl, float g,
    int L, int NBK, int Lb, int translen, int i0, int j0, int bi, int tlo, int thi, double safe, const float (*post)[16]) {
    const int lane = threadIdx.x, half = lane >> 5, l32 = lane & 31;
    const int bjA = (Lb - 1 - j0) / kBlk, bjB = bjA - 1;
    const int ia = i0 + l32 < Lb ? i0 + l32 : Lb - 1;
    const int pitch = translen - 1;
#pragma unroll 1
    for (int jh = 0; jh < 2; ++jh) {
        const int j = j0 + 32 * jh + l32, jb = j < Lb ? j : Lb - 1;
        const bool selA = (Lb - 1 - jb) / kBlk == bjA;
        const int dl = j - (i0 + 4 * half) - 1, pl = (i0 + 4 * half) * pitch + j - 1;
        auto valid = [&](int v) { return j < Lb && (unsigned)(dl - (8 * (v / 4) + (v % 4))) < (unsigned)translen; };
        auto index = [&](int v) { return pl + (8 * (v / 4) + (v % 4)) * pitch; };
        float e2[16], acc[16];   // E * log2(e) (-inf where there is no transition), sums
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            e2[v] = valid(v) ? to_float(lk[index(v)]) * kLog2e : DAGX_NEG_INF;
            acc[v] = ONLY_OVER ? post[jh][v] : 0.f;
        }
        // one step, given its block offsets (wave-uniform: ca = alpha block offset - Z; the two beta blocks' offsets) and
        // the step's residuals of this lane's column (rb) and row l32 (arow)
        auto one_step = [&](const double ca, const double cbA, const double cbB, const float rb, const float arow) __attribute__((always_inline)) {
            // beta side of the lane's column: residual + block offset + (alpha block offset - Z); -inf when dead
            const double kb = selA ? cbA : cbB;
            const double w = kb > (double)DAGX_NEG_INF ? (double)rb + (kb + ca) : (double)DAGX_NEG_INF;
            const int arow_bits = __builtin_bit_cast(int, arow);   // lane l32 (both halves) holds the residual of row i0 + l32
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = 8 * (v / 4) + (v % 4);                       // + 4 * half
                // (two reads of a fixed lane and a select: a cross-lane permute would make every one of the sixteen
                //  wait for its own round trip through the LDS crossbar)
                const float a_lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(arow_bits, row));
                const float a_hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(arow_bits, row + 4));
                const double ad = (double)(half ? a_hi : a_lo);
                acc[v] += fast_exp2(__builtin_fmaf((float)(w + ad), kLog2e, e2[v]));
            }
        };
        if constexpr (!ONLY_OVER) {
            for (int t = tlo; t <= thi; ++t) {
                const double ca = ao[t * NBK + bi] - Z;
                const double cbA = bo[(t + 1) * NBK + bjA];
                const double cbB = bjB >= 0 ? bo[(t + 1) * NBK + bjB] : (double)DAGX_NEG_INF;
                if (!(ca > (double)DAGX_NEG_INF) || !(fmax(cbA, cbB) > (double)DAGX_NEG_INF)) continue;   // wave-uniform
                one_step(ca, cbA, cbB, be_f[t * L + jb], al_f[t * L + ia]);
            }
        } else {
            auto uniform_of = [&](const double x, const int src) -> double {   // lane src's value, in scalar registers
                const long long bits = __builtin_bit_cast(long long, x);
                const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(bits & 0xffffffffLL), src);
                const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(bits >> 32), src);
                return __builtin_bit_cast(double, ((long long)hi << 32) | (long long)lo);
            };
            for (int g0 = tlo; g0 <= thi; g0 += kWave) {   // lane <-> step: which of these 64 steps were left out (as in step_scales)
                const bool live = g0 + lane <= thi;
                const int tl = live ? g0 + lane : thi;
                const double ca_l = ao[tl * NBK + bi] - Z, cbA_l = bo[(tl + 1) * NBK + bjA];
                const double cbB_l = bjB >= 0 ? bo[(tl + 1) * NBK + bjB] : (double)DAGX_NEG_INF;
                const double cbm = fmax(cbA_l, cbB_l);
                const bool dead = !live || !(ca_l > (double)DAGX_NEG_INF) || !(cbm > (double)DAGX_NEG_INF);
                unsigned long long over = __builtin_amdgcn_ballot_w64(!dead && !(ca_l + cbm <= safe));
                if (!over) continue;
                // the residual rows of a step are requested while the step before it is summed
                int k = __builtin_ctzll(over);
                float rb_n = be_f[(g0 + k) * L + jb], arow_n = al_f[(g0 + k) * L + ia];
                while (over) {
                    const int kc = k;
                    const float rb = rb_n, arow = arow_n;
                    over &= over - 1;
                    if (over) {
                        k = __builtin_ctzll(over);
                        rb_n = be_f[(g0 + k) * L + jb]; arow_n = al_f[(g0 + k) * L + ia];
                    }
                    one_step(uniform_of(ca_l, kc), uniform_of(cbA_l, kc), uniform_of(cbB_l, kc), rb, arow);
                }
            }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v)
            if (valid(v)) gl[index(v)] = from_float<TL>(g * acc[v]);
    }
}

template <typename TL>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(5, 5)))
void dag_grad_links_tiles_kernel(GradTileArgs a) {
    // (the streaming workgroups come last in the grid: dispatched first they delay the tiles, 44 us against 39)
    if ((int)blockIdx.x >= a.tile_blocks) { grad_side_jobs(a, (int)blockIdx.x - a.tile_blocks); return; }
    const int tile_id = (int)blockIdx.x;
    // Workgroup id -> (sample, tile half) with the sample varying fastest: consecutive ids go to different
    // XCDs, so every XCD gets whole samples (balanced work, and a sample's tables stay in one L2).
    const int b = tile_id % a.B, q = tile_id / a.B;
    const int ih = q & 1, tidx = q >> 1;
    const int bi = a.tile_bi[tidx], jt = a.tile_jt[tidx];
    const int lane = threadIdx.x;
    const int L = a.L, T = a.T, translen = a.translen, NBK = a.NBK;
    const int Lb = (int)a.out_len[b], Tb = (int)a.tgt_len[b];
    const double Z = a.logz[a.B + b];
    if (!lengths_ok(Lb, Tb, L, T) || Tb < 2 || !finite_d(Z)) return;
    const int i0 = bi * kBlk + 32 * ih, j0 = jt * kBlk;
    // no (i < j < L_b, j - i <= translen) in this tile
    if (i0 >= Lb - 1 || j0 >= Lb || j0 + kBlk - 1 <= i0 || j0 - (i0 + 31) > translen) return;
    // operand layout of the 32x32x2 MFMA: lanes 0..31 carry step t, lanes 32..63 step t+1
    const int half = lane >> 5, l32 = lane & 31;
    // beta blocks of this tile's columns: positions L_b-1-j run downwards, at most two blocks
    const int bjA = (Lb - 1 - j0) / kBlk;
    const int bjB = bjA - 1;
    // Rows >= L_b and columns >= L_b are read through clamped (in-bounds) indices and not masked:
    // whatever they contribute lands in accumulator rows / columns that the epilogue never writes out.
    const int ia = i0 + l32 < Lb ? i0 + l32 : Lb - 1;
    const int jb0 = j0 + l32 < Lb ? j0 + l32 : Lb - 1, jb1 = j0 + 32 + l32 < Lb ? j0 + 32 + l32 : Lb - 1;
    const bool selA0 = (Lb - 1 - jb0) / kBlk == bjA, selA1 = (Lb - 1 - jb1) / kBlk == bjA;
    const char *al = reinterpret_cast<const char *>(a.ahat + (int64_t)b * T * L);
    const char *be = reinterpret_cast<const char *>(a.bhat + (int64_t)b * T * L + L);   // beta of step t+1
    const double *ao = a.aoff + (int64_t)b * T * NBK, *bo = a.boff + (int64_t)b * T * NBK;
    // The tile's link values are needed only after the step loop.  Those of the first column half are
    // fetched now, straight into LDS (no registers held across the loop), so that this read overlaps
    // the loop; the second half is loaded while the first is being finished.  Element (i, j) of the
    // sample sits at index i * (translen - 1) + j - 1; invalid cells read element 0.
    //   value v of column half jh: row i0 + 8 (v / 4) + 4 half + v % 4, column j0 + 32 jh + l32
    __shared__ unsigned landing[16 * kWave];
    const TL *lk = static_cast<const TL *>(a.links) + (int64_t)b * L * translen;
    const unsigned landing_lds = (unsigned)reinterpret_cast<uintptr_t>(landing);
    const int pitch = translen - 1;
    int dl[2], pl[2];   // per lane and column half: d and element index of the lane's first row
    bool jok[2];
#pragma unroll
    for (int jh = 0; jh < 2; ++jh) {
        const int j = j0 + 32 * jh + l32;
        jok[jh] = j < Lb;
        dl[jh] = j - (i0 + 4 * half) - 1;
        pl[jh] = (i0 + 4 * half) * pitch + j - 1;
    }
    auto cell_valid = [&](int jh, int v) { return jok[jh] && (unsigned)(dl[jh] - (8 * (v / 4) + (v % 4))) < (unsigned)translen; };
    auto cell_index = [&](int jh, int v) { return pl[jh] + (8 * (v / 4) + (v % 4)) * pitch; };
#pragma unroll
    for (int v = 0; v < 16; ++v)
        dma_elem<TL>(landing_lds + (unsigned)v * (kWave * 4u), lk, cell_valid(0, v) ? (unsigned)cell_index(0, v) * (unsigned)sizeof(TL) : 0u);
    f32x16 c0, c1;   // column halves
#pragma unroll
    for (int r = 0; r < 16; ++r) { c0[r] = 0.f; c1[r] = 0.f; }
    const int slack = Lb - Tb;
    // alpha[t][i] is alive for i - slack <= t <= i; beta[t+1][j] for j - slack - 1 <= t <= j - 1
    int tlo = j0 - slack - 1; if (tlo < i0 - slack) tlo = i0 - slack; if (tlo < 0) tlo = 0;
    int thi = i0 + 31; if (thi > Tb - 2) thi = Tb - 2;
    // Scale factors of kGroup steps at a time, worked out with lane <-> step (float64 arithmetic once
    // per step) and kept in LDS in log2 units:
    //   [0]: on exp(alpha_hat);  [1] / [2]: on exp(beta_hat) for the two beta blocks of the columns.
    // Steps past thi get -inf everywhere: both factors become 0, whatever row was loaded for them.
    constexpr int kGroup = kWave;
    __shared__ float scales[3][kGroup];
    const double safe = safe_log_k(thi - tlo + 1);   // log K_t up to which a step goes through the matrix product
    bool unsafe = false;   // wave-uniform: some step of the tile has log K_t > safe; those steps are left out of the loop
    auto step_scales = [&](int t0) {
        const int sl = lane;
        const bool live = t0 + sl <= thi;
        const int t = live ? t0 + sl : thi;
        const double ca = ao[t * NBK + bi], cbA = bo[(t + 1) * NBK + bjA];
        const double cbB = bjB >= 0 ? bo[(t + 1) * NBK + bjB] : (double)DAGX_NEG_INF;
        const double cbm = fmax(cbA, cbB);
        bool dead = !live || !(ca > (double)DAGX_NEG_INF) || !(cbm > (double)DAGX_NEG_INF);
        const bool over = !dead && !((ca - Z) + cbm <= safe);   // (the same expression as in grad_tile_direct; a NaN counts)
        unsafe = unsafe || __builtin_amdgcn_ballot_w64(over) != 0;
        dead = dead || over;
        const double xm = dead ? 0.0 : (ca - Z) + cbm;
        double h = 0.5 * xm; if (h > 64.0) h = 64.0;
        __syncthreads();   // the previous group's reads are done
        {
            scales[0][sl] = dead ? DAGX_NEG_INF : (float)h * kLog2e;
            scales[1][sl] = !dead && cbA > (double)DAGX_NEG_INF ? (float)((cbA - cbm) + (xm - h)) * kLog2e : DAGX_NEG_INF;
            scales[2][sl] = !dead && cbB > (double)DAGX_NEG_INF ? (float)((cbB - cbm) + (xm - h)) * kLog2e : DAGX_NEG_INF;
        }
        __syncthreads();
    };
    const float *fa_p = &scales[0][half], *fb0_p = &scales[selA0 ? 1 : 2][half], *fb1_p = &scales[selA1 ? 1 : 2][half];
    // Step pairs are loaded kDepth pairs before they are used (with several waves sharing a SIMD that
    // is a few microseconds, enough for a miss): the address is a wave-uniform row
    // offset plus a per-lane constant.  All loads are unconditional and in bounds: a pair whose second
    // step is past thi reads the row of its first step twice (beta) or the row after thi (alpha, which
    // exists: thi + 1 <= T_b - 1), and pairs wholly past the end repeat the last one.
    constexpr int kDepth = 8;
    const unsigned va = (unsigned)(half * L + ia) * 4u;
    const unsigned vb0 = (unsigned)(half * L + jb0) * 4u, vb1 = (unsigned)(half * L + jb1) * 4u;
    const unsigned vb0_single = (unsigned)jb0 * 4u, vb1_single = (unsigned)jb1 * 4u;
    float ra[kDepth], rb0[kDepth], rb1[kDepth];
    auto issue = [&](int k, int t) {   // t: first step of the pair
        const int tb = t < thi ? t : thi;
        const bool full = tb < thi;
        const unsigned row = (unsigned)(tb * L) * 4u;   // wave-uniform
        ra[k] = *reinterpret_cast<const float *>(al + row + va);
        rb0[k] = *reinterpret_cast<const float *>(be + row + (full ? vb0 : vb0_single));
        rb1[k] = *reinterpret_cast<const float *>(be + row + (full ? vb1 : vb1_single));
    };
    auto consume = [&](int k, int idx) {   // idx: index of the pair's first step in its group
        const float ea = fast_exp2(__builtin_fmaf(ra[k], kLog2e, fa_p[idx]));
        const float eb0 = fast_exp2(__builtin_fmaf(rb0[k], kLog2e, fb0_p[idx]));
        const float eb1 = fast_exp2(__builtin_fmaf(rb1[k], kLog2e, fb1_p[idx]));
        c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(ea, eb0, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(ea, eb1, c1, 0, 0, 0);
    };
    if (tlo <= thi) {
#pragma unroll
        for (int k = 0; k < kDepth; ++k) issue(k, tlo + 2 * k);
        for (int g0 = tlo; g0 <= thi; g0 += kGroup) {
            step_scales(g0);
            // (the inner loop holds no loads but the ring's, so that the compiler can count them)
            const int gend = g0 + kGroup - 1 < thi ? g0 + kGroup - 1 : thi;
            for (int t = g0; t <= gend; t += 2 * kDepth) {
                const int idx0 = t - g0;                    // multiple of 16
#pragma unroll
                for (int k = 0; k < kDepth; ++k) {
                    consume(k, idx0 + 2 * k);               // pairs wholly past the end add zeros
                    issue(k, t + 2 * k + 2 * kDepth);
                    __builtin_amdgcn_sched_barrier(0);      // keep each refill where it is: kDepth - 1 pairs ahead of its use
                }
            }
        }
    }
    // epilogue: multiply by P = exp(E) and the upstream gradient, write the valid part of the tile
    const float g = a.grad_out[b * a.gstride];
    TL *gl = static_cast<TL *>(a.grad_links) + (int64_t)b * L * translen;
    wait_vmem_all();     // the link values of the first column half have landed
    __syncthreads();
    TL second[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) second[v] = lk[cell_valid(1, v) ? cell_index(1, v) : 0];
    auto link_of = [&](int jh, int v) -> float { return jh ? to_float(second[v]) : dma_decode<TL>(landing[v * kWave + lane]); };
    bool overflowed;
    {   // a sum that is not a finite number in a cell this wave writes: the bound rules that out for finite tables
        bool bad = false;
#pragma unroll
        for (int v = 0; v < 16; ++v)
            bad = bad || (cell_valid(0, v) && !(c0[v] <= 3.0e38f)) || (cell_valid(1, v) && !(c1[v] <= 3.0e38f));
        overflowed = __builtin_amdgcn_ballot_w64(bad) != 0;
    }
    if (__builtin_expect(overflowed, 0)) {   // a NaN in the tables: the whole tile, every step in the direct form
        grad_tile_direct<TL, false>(reinterpret_cast<const float *>(al), reinterpret_cast<const float *>(be), ao, bo, Z, lk, gl, g,
                                    L, NBK, Lb, translen, i0, j0, bi, tlo, thi, safe, nullptr);
        return;
    }
    // posterior sums of the lane's cells of one column half: the loop's sums times P = exp(E)
    auto posteriors = [&](auto all_valid, int jh, const f32x16 &c, float (&post)[16]) __attribute__((always_inline)) {
        // transitions too small for exp() in float32 take their factor through the logarithm of the sum
        bool tiny = false;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float e = link_of(jh, v);
            tiny = tiny || ((decltype(all_valid)::value || cell_valid(jh, v)) && e < -80.f && e > DAGX_NEG_INF);
        }
        const bool any_tiny = __builtin_amdgcn_ballot_w64(tiny) != 0;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const bool valid = decltype(all_valid)::value || cell_valid(jh, v);
            const float e = link_of(jh, v);
            post[v] = valid ? c[v] * fast_exp2(e * kLog2e) : 0.f;
            if (any_tiny && valid && e < -80.f) post[v] = (c[v] > 0.f && e > DAGX_NEG_INF) ? fast_exp2(__builtin_fmaf(e, kLog2e, fast_log2(c[v]))) : 0.f;
        }
    };
    if (__builtin_expect(unsafe, 0)) {   // the steps the loop left out, in the direct form, on top of the loop's sums
        float post[2][16];
        posteriors(std::false_type{}, 0, c0, post[0]);
        posteriors(std::false_type{}, 1, c1, post[1]);
        grad_tile_direct<TL, true>(reinterpret_cast<const float *>(al), reinterpret_cast<const float *>(be), ao, bo, Z, lk, gl, g,
                                   L, NBK, Lb, translen, i0, j0, bi, tlo, thi, safe, post);
        return;
    }
    auto finish = [&](auto all_valid, int jh, const f32x16 &c) {
        float post[16];
        posteriors(all_valid, jh, c, post);
#pragma unroll
        for (int v = 0; v < 16; ++v)
            if (decltype(all_valid)::value || cell_valid(jh, v)) gl[cell_index(jh, v)] = from_float<TL>(g * post[v]);
    };
#pragma unroll
    for (int jh = 0; jh < 2; ++jh) {
        const int jlo = j0 + 32 * jh;
        // every cell of the 32x32 block valid (wave-uniform): no per-element predicates
        const bool interior = jlo + 31 < Lb && jlo - (i0 + 31) - 1 >= 0 && jlo + 31 - i0 - 1 < translen;
        if (interior) finish(std::true_type{}, jh, jh ? c1 : c0);
        else finish(std::false_type{}, jh, jh ? c1 : c0);
    }
}


// ---- host side ------------------------------------------------------------------------------
static int check_common(const void *match, int mdt, const int64_t *ms, const void *links, int ldt,
                        const int64_t *ol, const int64_t *tl, int B, int T, int L, int translen, const char *who) {
    if (B < 0 || T < 1 || L < 1 || translen < 1) { set_error("%s: bad sizes B=%d T=%d L=%d translen=%d", who, B, T, L, translen); return DAGX_ERR_ARGUMENT; }
    if (B > 0 && (!match || !ms || !links || !ol || !tl)) { set_error("%s: null pointer argument", who); return DAGX_ERR_ARGUMENT; }
    if (mdt < DAGX_F32 || mdt > DAGX_BF16 || ldt < DAGX_F32 || ldt > DAGX_BF16) { set_error("%s: unsupported dtype", who); return DAGX_ERR_ARGUMENT; }
    if (L > 8192) { set_error("%s: graph size L=%d exceeds the supported 8192", who, L); return DAGX_ERR_UNSUPPORTED; }
    if (B > 65535 || T > 65535) { set_error("%s: B and T must not exceed 65535", who); return DAGX_ERR_UNSUPPORTED; }
    return DAGX_OK;
}


static bool force_exact() { return force_log_domain(); }

// ticket + launch counter (16 ints), 2*B*C progress words, B "left" counters, B risk words; rounded to 8 bytes
static size_t sweep_sync_ints(int B, int C) { return ((16 + (size_t)2 * B * C + (size_t)2 * B) + 1) & ~(size_t)1; }

size_t loss_fwd_workspace_bytes(int B, int T, int L, int translen) {
    (void)T;
    int C = groups_used(2 * ((B + 7) & ~7), L, translen, false);
    // ticket + progress words (rounded to 8 bytes), then the fast kernel's two read-outs per sample
    return C > 0 ? sweep_sync_ints(B, C) * sizeof(int) + (size_t)2 * B * sizeof(double) : 0;
}

size_t loss_bwd_workspace_bytes(int B) { (void)B; return 0; }

// The tile kernel's dynamic LDS (transpose patches while the tiles are staged, step buffers afterwards) exceeds the
// default limit: the limit is raised once per device and instantiation (not a call a graph capture may contain;
// dagx_prepare_device does it for every instantiation ahead of time).
constexpr size_t kPatchBytes = (size_t)kTileWaves * kBlk * (kBlk + 1) * sizeof(float);
template <bool WIDE> constexpr size_t tiles_lds_bytes() {
    return kPatchBytes > (size_t)StepLds<WIDE>::kStepFloats * sizeof(float) ? kPatchBytes : (size_t)StepLds<WIDE>::kStepFloats * sizeof(float);
}
template <typename TM, typename TL, bool WIDE>
static int prepare_tiles_kernel() {
    static std::atomic<unsigned long long> attr_set{0};   // per template instantiation: one bit per device
    int device = 0;
    (void)hipGetDevice(&device);
    const unsigned long long bit = 1ull << (device & 63);
    if (!(attr_set.load(std::memory_order_acquire) & bit)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(dag_sweep_tiles_kernel<TM, TL, WIDE>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)tiles_lds_bytes<WIDE>());
        if (e != hipSuccess) { set_error("dag_loss_fwd: cannot reserve %zu bytes of LDS: %s", tiles_lds_bytes<WIDE>(), hipGetErrorString(e)); return DAGX_ERR_LAUNCH; }
        attr_set.fetch_or(bit, std::memory_order_release);
    }
    return DAGX_OK;
}
template <typename TM>
static int prepare_tiles_kernels_of() {
    int rc = prepare_tiles_kernel<TM, float, false>();
    if (!rc) rc = prepare_tiles_kernel<TM, __half, false>();
    if (!rc) rc = prepare_tiles_kernel<TM, bf16_t, false>();
    if (!rc) rc = prepare_tiles_kernel<TM, float, true>();
    if (!rc) rc = prepare_tiles_kernel<TM, __half, true>();
    if (!rc) rc = prepare_tiles_kernel<TM, bf16_t, true>();
    return rc;
}

template <typename TM, typename TL>
static int launch_sweeps(SweepArgs a, hipStream_t st) {
    int C = force_exact() ? 0 : groups_used(2 * ((a.B + 7) & ~7), a.L, a.translen, false);
    // the tile kernel indexes match with 32-bit arithmetic
    const int64_t span = (int64_t)(a.T - 1) * (a.ms1 < 0 ? -a.ms1 : a.ms1) + (int64_t)(a.L - 1) * (a.ms2 < 0 ? -a.ms2 : a.ms2);
    if (span >= (1LL << 31) / (int64_t)sizeof(TM) || a.ms1 < 0 || a.ms2 < 0) C = 0;
    int rc;
    if (C == 0) {   // every sample goes to the log-domain kernel
        hipLaunchKernelGGL(dag_fill_int_kernel, dim3((a.B + 255) / 256), dim3(256), 0, st, a.flags, a.B, 1);
        if ((rc = check_launch("dag_fill"))) return rc;
    }
    if (C > 0) {
        a.zfast = reinterpret_cast<double *>(a.sync + sweep_sync_ints(a.B, C));
        // Two sweeps per sample whose read-outs bracket log Z.  With gradients they are the alpha sweep (rounding
        // up) and the beta sweep (rounding down; its read-out is the loss, as in fs_plugins/custom_ops/dag_loss.py:106-109).
        // Without, the reference runs the alpha sweep alone (dag_loss.cu:346-371); here a second alpha sweep that
        // rounds up rides along, so that the value returned is never one the linear domain has silently cut short.
        a.ndir = 2;
        a.rev[0] = 0; a.rev[1] = a.loss_dir ? 1 : 0;
        a.upper[0] = a.loss_dir ? 1 : 0; a.upper[1] = a.loss_dir ? 0 : 1;
        a.C = C;
        {
            const int W = (a.translen + kBlk - 1) / kBlk;
            int tmp[kTileCap + 2];
            for (int nb = 0; nb <= kMaxBlocksFast; ++nb) {
                partition_blocks(nb, W, C, tmp);
                for (int q = 0; q <= C && q < 12; ++q) a.gtab[nb][q] = (unsigned char)tmp[q];
            }
        }
        const int B8 = (a.B + 7) & ~7;
        if ((rc = prepare_tiles_kernel<TM, TL, false>()) || (rc = prepare_tiles_kernel<TM, TL, true>())) return rc;
        if (!float64_first()) {
            a.only_flagged = 0;
            hipLaunchKernelGGL((dag_sweep_tiles_kernel<TM, TL, false>), dim3(a.ndir * B8 * C), dim3(kTileWaves * kWave), tiles_lds_bytes<false>(), st, a);
            if ((rc = check_launch("dag_sweep_tiles"))) return rc;
        } else {   // the caller knows its inputs for sharply peaked: no float32 pass whose result would not stand
            hipLaunchKernelGGL(dag_mark_all_kernel, dim3((a.B + 255) / 256), dim3(256), 0, st, a.flags, a.B, a.sync);
            if ((rc = check_launch("dag_mark_all"))) return rc;
        }
        // the samples whose two read-outs did not agree, once more with float64 linear-domain numbers (the pipeline
        // words are zero again, as the first launch found them)
        a.only_flagged = 1;
        hipLaunchKernelGGL((dag_sweep_tiles_kernel<TM, TL, true>), dim3(a.ndir * B8 * C), dim3(kTileWaves * kWave), tiles_lds_bytes<true>(), st, a);
        if ((rc = check_launch("dag_sweep_tiles (wide)"))) return rc;
    }
    constexpr int NT = 1024;
    a.only_flagged = 1;
    const size_t lds = (size_t)a.L * 2 * sizeof(double);
    auto exact_kernel = dag_sweep_exact_kernel<TM, TL, NT>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(exact_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) { set_error("dag_loss_fwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); return DAGX_ERR_LAUNCH; }
    }
    hipLaunchKernelGGL(exact_kernel, dim3(a.B, a.loss_dir ? 2 : 1), dim3(NT), lds, st, a);
    return check_launch("dag_sweep_exact");
}

template <typename TM>
static int dispatch_links(int ldt, const SweepArgs &a, hipStream_t st) {
    switch (ldt) {
        case DAGX_F32: return launch_sweeps<TM, float>(a, st);
        case DAGX_F16: return launch_sweeps<TM, __half>(a, st);
        default: return launch_sweeps<TM, bf16_t>(a, st);
    }
}

struct BwdArgs {
    const float *go; int64_t gs;
    const float *ahat, *bhat; const double *aoff, *boff, *logz;
    const int64_t *ol, *tl; int B, T, L, translen, NBK;
};

static bool grad_tiles_apply(int L) { return !force_exact() && (L + kBlk - 1) / kBlk <= kMaxBlocksFast; }

// what has to be cleared in front of the grad_links tile kernel
static ZeroJob make_zero_job(const BwdArgs &g, void *gl, size_t elem) {
    int chunks = g.L < 32 ? g.L : 32;
    const int rows = (g.L + chunks - 1) / chunks;
    chunks = (g.L + rows - 1) / rows;
    return ZeroJob{static_cast<unsigned char *>(gl), (int)elem, g.ol, g.tl, g.logz, g.B, g.T, g.L, g.translen,
                   rows, chunks, g.B * chunks};
}

template <typename TM>
static int launch_grad_match(const BwdArgs &g, const void *match, const int64_t *ms, void *gm, const ZeroJob &zero, hipStream_t st) {
    const int64_t blocks = (int64_t)zero.blocks + (int64_t)((g.L + 255) / 256) * g.T * g.B;
    if (blocks > 0x7fffffffLL) { set_error("dag_loss_bwd: B*T*L too large for one launch"); return DAGX_ERR_UNSUPPORTED; }
    hipLaunchKernelGGL((dag_grad_match_kernel<TM>), dim3((unsigned)blocks), dim3(256), 0, st, g.go, g.gs,
                       g.ahat, g.bhat, g.aoff, g.boff, g.logz, static_cast<const TM *>(match), ms[0], ms[1], ms[2],
                       g.ol, g.tl, g.B, g.T, g.L, g.NBK, static_cast<TM *>(gm), zero);
    return check_launch("dag_grad_match");
}

// match / ms / match_dtype / gm: grad_match to be computed in the same launch as the tiles (gm == nullptr: not asked for,
// or already done by a launch of its own)
template <typename TL>
static int launch_grad_links(const BwdArgs &g, const void *links, void *gl, const void *match, const int64_t *ms,
                             int match_dtype, void *gm, hipStream_t st) {
    if (grad_tiles_apply(g.L)) {
        // block-scaled tiles (with their own direct-form redo); zeros where no tile writes and grad_match from
        // workgroups of the same launch
        GradTileArgs ta{g.go, g.gs, g.ahat, g.bhat, g.aoff, g.boff, g.logz, links, gl, g.ol, g.tl,
                        g.B, g.T, g.L, g.translen, g.NBK};
        ta.zero = make_zero_job(g, gl, sizeof(TL));
        ta.match = match; ta.match_dtype = match_dtype; ta.grad_match = gm;
        if (gm) { ta.ms0 = ms[0]; ta.ms1 = ms[1]; ta.ms2 = ms[2]; }
        const int NB = (g.L + kBlk - 1) / kBlk;
        int W = (g.translen + kBlk - 1) / kBlk; if (W > NB - 1) W = NB - 1;
        ta.ntile = 0;
        for (int bi = 0; bi < NB; ++bi)
            for (int jt = bi; jt <= bi + W && jt < NB; ++jt) { ta.tile_bi[ta.ntile] = (unsigned char)bi; ta.tile_jt[ta.ntile] = (unsigned char)jt; ++ta.ntile; }
        ta.tile_blocks = 2 * ta.ntile * g.B;   // two row halves per tile
        const int64_t match_blocks = gm ? (int64_t)((g.L + 255) / 256) * g.T * g.B : 0;
        const int64_t blocks = (int64_t)ta.tile_blocks + ta.zero.blocks + match_blocks;
        if (blocks > 0x7fffffffLL) { set_error("dag_loss_bwd: B*T*L too large for one launch"); return DAGX_ERR_UNSUPPORTED; }
        ta.match_blocks = (int)match_blocks;
        hipLaunchKernelGGL((dag_grad_links_tiles_kernel<TL>), dim3((unsigned)blocks), dim3(kWave), 0, st, ta);
        return check_launch("dag_grad_links_tiles");
    }
    // direct (log-domain) form: graphs beyond the tile kernels, or the log-domain-only mode
    constexpr int RI = 32;
    hipLaunchKernelGGL((dag_grad_links_kernel<TL, RI>), dim3((g.translen + 63) / 64, (g.L + RI - 1) / RI, g.B), dim3(256), 0, st,
                       g.go, g.gs, g.ahat, g.bhat, g.aoff, g.boff, g.logz, static_cast<const TL *>(links), g.ol, g.tl,
                       g.B, g.T, g.L, g.translen, g.NBK, static_cast<TL *>(gl));
    return check_launch("dag_grad_links");
}

}  // namespace dagx

using namespace dagx;


static int loss_fwd_impl(const void *match, int match_dtype, const int64_t match_strides[3],
                         const void *links, int links_dtype,
                         const int64_t *out_len, const int64_t *tgt_len,
                         int B, int T, int L, int translen,
                         float *alpha_hat, float *beta_hat, double *alpha_off, double *beta_off,
                         double *logz, float *loss, int *sample_flags, int require_gradient,
                         void *workspace, size_t workspace_bytes, void *stream) {
    int rc = check_common(match, match_dtype, match_strides, links, links_dtype, out_len, tgt_len, B, T, L, translen, "dag_loss_fwd");
    if (rc) return rc;
    if (B == 0) return DAGX_OK;                 // an empty batch owns no memory: nothing to check or launch
    if (!alpha_hat || !beta_hat || !alpha_off || !beta_off || !logz || !loss || !sample_flags) { set_error("dag_loss_fwd: an output pointer is null"); return DAGX_ERR_ARGUMENT; }
    size_t need = loss_fwd_workspace_bytes(B, T, L, translen);
    if (need > 0 && (!workspace || workspace_bytes < need)) { set_error("dag_loss_fwd: workspace of %zu bytes required, %zu given", need, workspace_bytes); return DAGX_ERR_WORKSPACE; }
    SweepArgs a{};
    a.match = match; a.ms0 = match_strides[0]; a.ms1 = match_strides[1]; a.ms2 = match_strides[2];
    a.links = links; a.out_len = out_len; a.tgt_len = tgt_len;
    a.B = B; a.T = T; a.L = L; a.translen = translen; a.NBK = (L + kBlk - 1) / kBlk;
    a.hat[0] = alpha_hat; a.hat[1] = beta_hat; a.off[0] = alpha_off; a.off[1] = beta_off;
    a.logz = logz; a.loss = loss; a.loss_dir = require_gradient ? 1 : 0; a.flags = sample_flags; a.sync = static_cast<int *>(workspace);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (match_dtype) {
        case DAGX_F32: return dispatch_links<float>(links_dtype, a, st);
        case DAGX_F16: return dispatch_links<__half>(links_dtype, a, st);
        default: return dispatch_links<bf16_t>(links_dtype, a, st);
    }
}

extern "C" int dagx_loss_fwd(const void *match, int match_dtype, const int64_t match_strides[3],
                             const void *links, int links_dtype,
                             const int64_t *out_len, const int64_t *tgt_len,
                             int B, int T, int L, int translen,
                             float *alpha_hat, float *beta_hat, double *alpha_off, double *beta_off,
                             double *logz, float *loss, int *sample_flags, int require_gradient,
                             void *workspace, size_t workspace_bytes, void *stream) {
    return loss_fwd_impl(match, match_dtype, match_strides, links, links_dtype, out_len, tgt_len, B, T, L, translen,
                         alpha_hat, beta_hat, alpha_off, beta_off, logz, loss, sample_flags, require_gradient,
                         workspace, workspace_bytes, stream);
}

// ---- the forward for callers that cannot allocate ------------------------------------------------------
// The pipeline words and read-outs of the tile sweeps (what dagx_loss_fwd takes as `workspace`) in a
// device array owned by the library: every GPU the library runs on holds its own copy until the process
// ends.  Zero when the code object is loaded; the sweep kernel leaves every word it used zero again.
constexpr size_t kScratchBytes = 128 * 1024;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (looked up once per device; in host code the
// array's name is only a handle for this lookup, never an address a kernel may be given).
static int scratch_of_current_device(void **out) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) { set_error("dag_loss_fwd_noalloc: hipGetDevice failed: %s", hipGetErrorString(e)); return DAGX_ERR_LAUNCH; }
    if (device < 0 || device >= kMaxDevices) { set_error("dag_loss_fwd_noalloc: device index %d not supported (max %d)", device, kMaxDevices - 1); return DAGX_ERR_UNSUPPORTED; }
    void *p = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) { set_error("dag_loss_fwd_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e)); return DAGX_ERR_LAUNCH; }
        g_scratch_ptr[device].store(p, std::memory_order_release);   // a concurrent first call stores the same address
    }
    *out = p;
    return DAGX_OK;
}

extern "C" size_t dagx_loss_fwd_noalloc_max_bytes(void) { return kScratchBytes; }

// Everything the forward entry points do once per device, done now: the LDS limit of every instantiation of the tile
// kernel and the address of the built-in scratch array.  After it, dagx_loss_fwd / dagx_loss_fwd_noalloc on this
// device make kernel launches only (for L <= 3072), which is what a stream capture may hold.
extern "C" int dagx_prepare_device(void) {
    int rc = prepare_tiles_kernels_of<float>();
    if (!rc) rc = prepare_tiles_kernels_of<__half>();
    if (!rc) rc = prepare_tiles_kernels_of<bf16_t>();
    void *ptr = nullptr;
    if (!rc) rc = scratch_of_current_device(&ptr);
    return rc;
}

// Zero-fill of a workspace for dagx_loss_fwd (a kernel launch on `stream`; needed once per buffer, before its first use).
extern "C" int dagx_loss_fwd_init_workspace(void *workspace, size_t workspace_bytes, void *stream) {
    if (workspace_bytes == 0) return DAGX_OK;
    if (!workspace || (workspace_bytes & 3) || (reinterpret_cast<uintptr_t>(workspace) & 7)) { set_error("dag_loss_fwd_init_workspace: needs an 8-byte aligned buffer of a multiple of 4 bytes"); return DAGX_ERR_ARGUMENT; }
    const size_t n = workspace_bytes / 4;
    if (n > 0x7fffffffu) { set_error("dag_loss_fwd_init_workspace: buffer too large"); return DAGX_ERR_ARGUMENT; }
    hipLaunchKernelGGL(dag_fill_int_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<int *>(workspace), (int)n, 0);
    return check_launch("dag_fill");
}

extern "C" int dagx_loss_fwd_noalloc(const void *match, int match_dtype, const int64_t match_strides[3],
                                     const void *links, int links_dtype,
                                     const int64_t *out_len, const int64_t *tgt_len,
                                     int B, int T, int L, int translen,
                                     float *alpha_hat, float *beta_hat, double *alpha_off, double *beta_off,
                                     double *logz, float *loss, int *sample_flags, int require_gradient,
                                     void *stream) {
    if (B < 0 || T < 1 || L < 1 || translen < 1) { set_error("dag_loss_fwd_noalloc: bad sizes B=%d T=%d L=%d translen=%d", B, T, L, translen); return DAGX_ERR_ARGUMENT; }
    const size_t need = loss_fwd_workspace_bytes(B, T, L, translen);
    if (need > kScratchBytes) {
        set_error("dag_loss_fwd_noalloc: B=%d, L=%d needs %zu bytes of pipeline words, the built-in scratch holds %zu "
                  "(use dagx_loss_fwd with a caller workspace)", B, L, need, kScratchBytes);
        return DAGX_ERR_UNSUPPORTED;
    }
    void *ptr = nullptr;
    if (need > 0) {
        const int rc = scratch_of_current_device(&ptr);
        if (rc) return rc;
    }
    return loss_fwd_impl(match, match_dtype, match_strides, links, links_dtype, out_len, tgt_len, B, T, L, translen,
                         alpha_hat, beta_hat, alpha_off, beta_off, logz, loss, sample_flags, require_gradient,
                         ptr, need > 0 ? kScratchBytes : 0, stream);
}

extern "C" int dagx_loss_bwd(const float *grad_out, int64_t grad_out_stride,
                             const float *alpha_hat, const float *beta_hat,
                             const double *alpha_off, const double *beta_off, const double *logz,
                             const int *sample_flags,
                             const void *match, int match_dtype, const int64_t match_strides[3],
                             const void *links, int links_dtype,
                             const int64_t *out_len, const int64_t *tgt_len,
                             int B, int T, int L, int translen,
                             void *grad_match, void *grad_links,
                             void *workspace, size_t workspace_bytes, void *stream) {
    int rc = check_common(match, match_dtype, match_strides, links, links_dtype, out_len, tgt_len, B, T, L, translen, "dag_loss_bwd");
    if (rc) return rc;
    if (B == 0) return DAGX_OK;
    if (!grad_out || !alpha_hat || !beta_hat || !alpha_off || !beta_off || !logz) { set_error("dag_loss_bwd: a saved-state pointer is null"); return DAGX_ERR_ARGUMENT; }
    (void)workspace; (void)workspace_bytes; (void)sample_flags;   // the backward needs no scratch
    hipStream_t st = static_cast<hipStream_t>(stream);
    BwdArgs g{grad_out, grad_out_stride, alpha_hat, beta_hat, alpha_off, beta_off, logz, out_len, tgt_len,
              B, T, L, translen, (L + kBlk - 1) / kBlk};
    // With both gradients asked for and the tile kernel in charge, grad_match rides in its launch.
    const bool together = grad_match && grad_links && grad_tiles_apply(L);
    if (grad_match && !together) {
        ZeroJob zero{};
        switch (match_dtype) {
            case DAGX_F32: rc = launch_grad_match<float>(g, match, match_strides, grad_match, zero, st); break;
            case DAGX_F16: rc = launch_grad_match<__half>(g, match, match_strides, grad_match, zero, st); break;
            default: rc = launch_grad_match<bf16_t>(g, match, match_strides, grad_match, zero, st); break;
        }
        if (rc) return rc;
    }
    if (grad_links) {
        switch (links_dtype) {
            case DAGX_F32: rc = launch_grad_links<float>(g, links, grad_links, match, match_strides, match_dtype, together ? grad_match : nullptr, st); break;
            case DAGX_F16: rc = launch_grad_links<__half>(g, links, grad_links, match, match_strides, match_dtype, together ? grad_match : nullptr, st); break;
            default: rc = launch_grad_links<bf16_t>(g, links, grad_links, match, match_strides, match_dtype, together ? grad_match : nullptr, st); break;
        }
    }
    return rc;
}

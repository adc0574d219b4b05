// Best alignment on gfx950: max-semiring sweep with back-pointers and an on-GPU backtrack.
//
//   A[t][j] = max_{i<j, j-i<=translen} fl32(A[t-1][i] + E[i][j]) + match[t][j]   (two fp32 roundings)
//   back[t][j] = the smallest i attaining the max; backtrack from (T_b-1, L_b-1).
//
// Two implementations:
//  * dag_align_tiles_kernel + dag_backtrack_kernel (L <= 1024): the sweep keeps E as 64x64 register
//    tiles and evaluates a step with one DPP-broadcast add and one max per (i, j) pair, spread over
//    the same pipeline of workgroups as the loss sweeps; it stores only the score table.  The
//    backtrack (one wave per sample) then re-derives, for the T_b cells on the path only, the
//    lowest predecessor index attaining the stored maximum.
//  * dag_align_kernel: one workgroup per sample, thread <-> node j scanning its predecessors in
//    ascending order with a strict '>' (back-pointers in LDS when T*L fits, else in the caller's
//    workspace).  Handles any L <= 8192; the backtrack kernel uses the same code for the samples that the
//    pipeline gave up on.
// Both evaluate fl32(A + E) then + match, so their scores -- and therefore the paths -- are
// bit-identical to the torch-native rule.
#include "dag_tiles.h"

namespace dagx {

struct AlignArgs {
    const void *match; int64_t ms0, ms1, ms2;
    const void *links;
    const int64_t *out_len, *tgt_len;
    int B, T, L, translen;
    int64_t *path;
    int32_t *trace_ws;  // [B][T][L] when the LDS variant is not used
};

// One sample by one workgroup of NT threads; lds_a: 2*L floats, then (TRACE_LDS) T*L uint16.
template <typename TM, typename TL, int NT, bool TRACE_LDS>
__device__ __forceinline__ void align_one_sample(const AlignArgs &a, const int b, float *lds_a) {
    const int tid = threadIdx.x;
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

    // A team of kTeam lanes <-> node j of the band; the team's lanes deal the predecessors i among themselves
    // (lane q takes i = ilo + q, ilo + q + kTeam, ...), R of them in flight per lane, and merge their
    // (best score, lowest index that has it) pairs by shuffles.  Nodes go to the teams round robin, which mixes
    // nodes with few and with many predecessors in every team.  Cells outside the band are never on a path:
    // their trace entries stay unwritten.
    constexpr int kTeam = 8, R = 8;
    const int team = tid / kTeam, sub = tid % kTeam;
    const unsigned rs = (unsigned)(translen - 1);   // E[i][j-i-1] sits at links[i*(translen-1) + j-1]: 32-bit offsets
    for (int t = 1; t < Tb; ++t) {
        const int jhi = slack + t;
        for (int j = tid; j < L; j += NT)
            if (j < t || j > jhi) fcur[j] = DAGX_NEG_INF;
        for (int j = t + team; j <= jhi; j += NT / kTeam) {
            const float mj = to_float(match[(int64_t)t * a.ms1 + (int64_t)j * a.ms2]);
            int ilo = j - translen; if (ilo < t - 1) ilo = t - 1;
            float best = DAGX_NEG_INF;
            int arg = ilo;
            const unsigned o_last = (unsigned)(j - 1) * (unsigned)translen;   // the offset of i = j-1, the largest
            unsigned o = (unsigned)(ilo + sub) * rs + (unsigned)(j - 1);
            for (int i0 = ilo + sub; i0 < j; i0 += kTeam * R, o += kTeam * R * rs) {
                float e[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const unsigned oc = o + (unsigned)(r * kTeam) * rs;
                    e[r] = to_float(links[oc < o_last ? oc : o_last]);
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const int i = i0 + r * kTeam;
                    const float x = i < j ? fprev[i < j ? i : j - 1] + e[r] : DAGX_NEG_INF;   // (index clamped: read, then selected)
                    if (x > best) { best = x; arg = i; }
                }
            }
#pragma unroll
            for (int w = kTeam / 2; w > 0; w >>= 1) {
                const float bo = __shfl_xor(best, w, kWave);
                const int ao = __shfl_xor(arg, w, kWave);
                if (bo > best || (bo == best && ao < arg)) { best = bo; arg = ao; }
            }
            if (sub == 0) {
                fcur[j] = best + mj;
                if (TRACE_LDS) tr_lds[(size_t)t * L + j] = (uint16_t)arg;
                else tr_glb[(int64_t)t * L + j] = arg;
            }
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

template <typename TM, typename TL, int NT, bool TRACE_LDS>
__global__ __launch_bounds__(NT) void dag_align_kernel(AlignArgs a) {
    extern __shared__ float lds_a[];
    align_one_sample<TM, TL, NT, TRACE_LDS>(a, blockIdx.x, lds_a);
}


// ================================================================================================
// Tile-resident max-plus sweep
// ================================================================================================

// best = max(best, max_{r<16} (a[lane r of this 16-lane row] + e[r])): two sums, then one three-way maximum
// (24 instructions for 16 rows instead of 32; a maximum does not round, so the result is the same bit for bit)
__device__ __forceinline__ void maxplus16_rowbcast(float &best, float av, const float *e) {
    float t1, t2;
    asm("s_nop 1\n\t"
        "v_add_f32_dpp %1, %3, %4 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %2, %3, %5 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_max3_f32 %0, %0, %1, %2\n\t"
        "v_add_f32_dpp %1, %3, %6 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %2, %3, %7 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
        "v_max3_f32 %0, %0, %1, %2\n\t"
        "v_add_f32_dpp %1, %3, %8 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %2, %3, %9 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
        "v_max3_f32 %0, %0, %1, %2\n\t"
        "v_add_f32_dpp %1, %3, %10 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %2, %3, %11 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
        "v_max3_f32 %0, %0, %1, %2\n\t"
        "v_add_f32_dpp %1, %3, %12 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %2, %3, %13 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
        "v_max3_f32 %0, %0, %1, %2\n\t"
        "v_add_f32_dpp %1, %3, %14 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %2, %3, %15 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
        "v_max3_f32 %0, %0, %1, %2\n\t"
        "v_add_f32_dpp %1, %3, %16 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %2, %3, %17 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
        "v_max3_f32 %0, %0, %1, %2\n\t"
        "v_add_f32_dpp %1, %3, %18 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %2, %3, %19 row_newbcast:15 row_mask:0xf bank_mask:0xf\n\t"
        "v_max3_f32 %0, %0, %1, %2"
        : "+v"(best), "=&v"(t1), "=&v"(t2)
        : "v"(av), "v"(e[0]), "v"(e[1]), "v"(e[2]), "v"(e[3]), "v"(e[4]), "v"(e[5]), "v"(e[6]), "v"(e[7]),
          "v"(e[8]), "v"(e[9]), "v"(e[10]), "v"(e[11]), "v"(e[12]), "v"(e[13]), "v"(e[14]), "v"(e[15]));
}

__device__ __forceinline__ float max3(float a, float b, float c) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

// max_{r<64} (a[r] + tile.p[r]); lane l holds a[l & 15], a[16 + (l & 15)], a[32 + (l & 15)], a[48 + (l & 15)]
__device__ __forceinline__ float tile_maxplus(const Tile &t, float a0, float a1, float a2, float a3) {
    float b0 = DAGX_NEG_INF, b1 = DAGX_NEG_INF;
    maxplus16_rowbcast(b0, a0, t.p);
    maxplus16_rowbcast(b1, a1, t.p + 16);
    maxplus16_rowbcast(b0, a2, t.p + 32);
    maxplus16_rowbcast(b1, a3, t.p + 48);
    return fmaxf(b0, b1);
}

// bytes per row of the source-block table (rows padded to 16 bytes)
__host__ __device__ static inline int srcblk_pitch(int L) { return (L + 15) & ~15; }

static int align_groups(int B, int L, int translen) { return groups_used((B + 7) & ~7, L, translen, true); }

struct AlignTileArgs {
    const void *match; int64_t ms0, ms1, ms2;
    const void *links;
    const int64_t *out_len, *tgt_len;
    int B, T, L, translen;
    float *table;     // [B][T][L] best score of every cell, by node
    unsigned char *srcblk;   // [B][T][pitch] block of 64 nodes that holds the best predecessor of every cell (the lowest such block); 16-byte aligned rows
    int *sync;        // [0] ticket counter, [16 + b*C + group] progress
    int *flags;       // [B] set when the pipeline gave up on a sample
    int C;
    int mcap;         // match row read at step s: min(s, mcap) (T-1 for the alignment: every step its own row)
    int decode;       // Viterbi decoding: every sample runs all T steps (tgt_len is not read) and no cell is
                      // pruned for being too far from the last node -- a path may end at any step
    unsigned char gtab[kMaxBlocksFast + 1][12];
};

// Same workgroup pipeline as the loss sweeps (tickets, one-way hand-over through the table with
// agent-scope accesses, bounded waits), in the (max, +) semiring and without any rescaling: the
// table holds the plain fp32 scores.
template <typename TM, typename TL>
__global__ __launch_bounds__(kTileWaves * kWave) void dag_align_tiles_kernel(AlignTileArgs a) {
    __shared__ float abuf[2][kMaxBlocksFast][kBlk];   // scores of the previous / next step, by node
    // tile results: the tiles of an owned block lie in consecutive rows that start at a multiple of eight, and the rows
    // behind them, up to the next multiple of eight, hold -inf for good: the owner reads whole eights without a test
    constexpr int kPartRows = kTileCap + 7 * kMaxBlocksFast;
    __shared__ float part[kPartRows][kBlk];
    // landing areas of the asynchronous global -> LDS copies (one slot per consuming wave), double-buffered by step parity
    __shared__ unsigned stage_m[2][kTileWaves][2][kBlk];   // match rows of the wave's own blocks (raw elements)
    __shared__ float stage_f[2][kTileWaves][2][kBlk];      // table rows of the wave's foreign blocks
    __shared__ int stage_p[2][kBlk];                        // snapshots of the progress word of the group below
    __shared__ int gstart[kTileCap + 2];
    __shared__ int s_ticket, s_abort;

    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int C = a.C;
    if (tid == 0) { s_ticket = atomicAdd(a.sync, 1); s_abort = 0; }
    __syncthreads();
    const int k = __builtin_amdgcn_readfirstlane(s_ticket);
    const int B8 = (a.B + 7) & ~7;
    // first group 0 of every sample, then every group 1, ... (see the loss sweep kernel: producers hold smaller tickets,
    // and what the dispatcher reaches last are consumers); the groups of a sample are a multiple of 8 tickets apart
    const int g = k / B8;
    const int b = ((k / 8) % (B8 / 8)) * 8 + (k % 8);
    if (g >= C || b >= a.B) return;

    const int L = a.L, T = a.T, translen = a.translen;
    const int Lb = (int)a.out_len[b], Tb = a.decode ? T : (int)a.tgt_len[b];
    if (!(Tb >= 1 && Lb >= 1 && Tb <= T && Lb <= L && (a.decode || Tb <= Lb))) return;   // the backtrack sees the lengths too
    const TM *match = static_cast<const TM *>(a.match) + (int64_t)b * a.ms0;
    const TL *links = static_cast<const TL *>(a.links) + (int64_t)b * L * translen;
    float *table = a.table + (int64_t)b * T * L;
    const int spitch = srcblk_pitch(L);
    unsigned char *srcblk = a.srcblk + (int64_t)b * T * spitch;
    int *prog = a.sync + 16 + b * C;

    const int slack = a.decode ? L : Lb - Tb;
    const int mcap = a.mcap;
    const int NBb = (Lb + kBlk - 1) / kBlk;
    const int W = (translen + kBlk - 1) / kBlk;
    if (tid <= C) gstart[tid] = a.gtab[NBb][tid];
    __syncthreads();
    const int jb0 = __builtin_amdgcn_readfirstlane(gstart[g]), jb1 = __builtin_amdgcn_readfirstlane(gstart[g + 1]);
    int last_group = 0;
    for (int q = 0; q < C; ++q) if (gstart[q + 1] > gstart[q]) last_group = q;
    last_group = __builtin_amdgcn_readfirstlane(last_group);
    if (jb0 >= jb1) return;
    const int nblk = jb1 - jb0;
    const int flo = tile_ilo(jb0, W);
    const bool producer = g < last_group;
    const bool consumer = flo < jb0;

    int ntile = 0;
    for (int Jb = jb0; Jb < jb1; ++Jb) ntile += Jb - tile_ilo(Jb, W) + 1;
    // The last wave is the fetcher (see the loss sweep kernel) and takes tiles only when the others cannot
    // hold them all; the tiles are dealt out evenly, the odd ones first to wave 3 (the fetcher's SIMD).
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
    int my_I[kTilesPerWave], my_J[kTilesPerWave], my_q[kTilesPerWave];
#pragma unroll
    for (int sl = 0; sl < kTilesPerWave; ++sl) { my_I[sl] = -1; my_J[sl] = -1; my_q[sl] = -1; }
    {   // (my_q: the row of the tile's result, see 'part')
        int q = 0, row0 = 0;
        for (int Jb = jb0; Jb < jb1; ++Jb) {
            for (int I = tile_ilo(Jb, W); I <= Jb; ++I, ++q) {
                const int sl = q - my_first;
                if (sl >= 0 && sl < my_count) {
#pragma unroll
                    for (int u = 0; u < kTilesPerWave; ++u)
                        if (u == sl) { my_I[u] = I; my_J[u] = Jb; my_q[u] = row0 + I - tile_ilo(Jb, W); }
                }
            }
            row0 += (Jb - tile_ilo(Jb, W) + 1 + 7) & ~7;
        }
    }
    Tile t0, t1, t2;
    if (my_q[0] >= 0) load_tile<false, 16>(t0, links, my_I[0], my_J[0], lane, 0, Lb, translen, nullptr, 0.f);
    if (my_q[1] >= 0) load_tile<false, 16>(t1, links, my_I[1], my_J[1], lane, 0, Lb, translen, nullptr, 0.f);
    if (my_q[2] >= 0) load_tile<false, 16>(t2, links, my_I[2], my_J[2], lane, 0, Lb, translen, nullptr, 0.f);

    const char *table_c = reinterpret_cast<const char *>(table);
    const char *match_c = reinterpret_cast<const char *>(match);
    auto cell = [&](int trow, int node) -> float * {
        return reinterpret_cast<float *>(const_cast<char *>(table_c) + (unsigned)(trow * L + node) * 4u);
    };
    const int ms1 = (int)a.ms1, ms2 = (int)a.ms2;   // the host checked that match indices fit 32 bits
    auto match_at = [&](int trow, int node) -> float {
        return to_float(*reinterpret_cast<const TM *>(match_c + (unsigned)(trow * ms1 + node * ms2) * (unsigned)sizeof(TM)));
    };

    // step 0: node 0 holds match[0][0] (even if that is -inf), everything else -inf
    const float m0 = match_at(0, 0);
    for (int q = tid; q < kMaxBlocksFast * kBlk; q += kTileWaves * kWave) {
        abuf[0][q / kBlk][q % kBlk] = q == 0 ? m0 : DAGX_NEG_INF;
        abuf[1][q / kBlk][q % kBlk] = DAGX_NEG_INF;
    }
    for (int q = tid; q < kPartRows * kBlk; q += kTileWaves * kWave) part[q / kBlk][q % kBlk] = DAGX_NEG_INF;
    for (int ob = wave; ob < nblk; ob += kTileWaves) {
        const int p = (jb0 + ob) * kBlk + lane;
        if (p < Lb) store_agent(cell(0, p), p == 0 ? m0 : DAGX_NEG_INF);
    }
    // ---- staging slots (see the loss sweep kernel): match rows of own blocks wave and wave + 8, table
    //      rows of foreign blocks flo + wave and flo + wave + 8, all filled by the fetcher ----
    constexpr int kFetchSlots = 2;
    int f_blk[kFetchSlots];
#pragma unroll
    for (int u = 0; u < kFetchSlots; ++u) {   // dealt from the last wave down: the first waves are the ones that own blocks
        const int fb = flo + (kTileWaves - 1 - wave) + kTileWaves * u;
        f_blk[u] = fb < jb0 ? fb : -1;
    }
    const int *below = prog + (g > 0 ? g - 1 : 0);
    auto lds_addr = [&](const void *p) -> unsigned { return (unsigned)reinterpret_cast<uintptr_t>(p); };
    const bool fetcher = wave == kTileWaves - 1;
    int seen = 0;   // last progress value of the group below that the fetcher has read
    // The fetcher works one step ahead, as in the loss sweep: in phase A of step s it waits for what it requested
    // a step ago (the rows phase B of step s reads), then requests the match rows of step s + 1, the foreign table
    // rows of step s + 1 if the snapshot of the producer's progress word (requested a step ago) shows them
    // published, and the next snapshot.  Only when the producer is less than two steps ahead does it poll the word
    // and fetch in the same step (one memory round trip inside phase A, which used to be every step's price).
#define DAGX_STAMP(COND, SLOT)
    int rows_issued = 0;   // the foreign table rows of steps <= rows_issued have been requested
    auto issue_match = [&](const int s2, const int lane) __attribute__((always_inline)) {
        const int par = s2 & 1;
        const TM *mrow = reinterpret_cast<const TM *>(match_c + (unsigned)((s2 < mcap ? s2 : mcap) * ms1) * (unsigned)sizeof(TM));
        for (int ob = 0; ob < nblk; ++ob) {
            const int pm = (jb0 + ob) * kBlk + lane, pmc = pm < Lb ? pm : Lb - 1;
            dma_elem<TM>(lds_addr(&stage_m[par][ob & (kTileWaves - 1)][ob / kTileWaves][0]), mrow, (unsigned)(pmc * ms2) * (unsigned)sizeof(TM));
        }
    };
    auto issue_rows = [&](const int s2, const int lane) __attribute__((always_inline)) {
        const int par = s2 & 1;
        for (int fb = flo; fb < jb0; ++fb) {
            const int q = fb - flo, pf = fb * kBlk + lane, pfc = pf < Lb ? pf : Lb - 1;
            dma_dword_agent(lds_addr(&stage_f[par][kTileWaves - 1 - (q & (kTileWaves - 1))][q / kTileWaves][0]), table_c + (unsigned)(s2 * L) * 4u, (unsigned)pfc * 4u);
        }
        rows_issued = s2;
    };
    auto fetch_step = [&](const int s) __attribute__((always_inline)) {
        // (the fetcher's lane arithmetic is redone every step, on purpose: computed ahead of the loop over the steps it
        //  would hold registers that the tiles need)
        int ln = lane;
        asm volatile("" : "+v"(ln));
        wait_vmem_all();   // everything requested a step ago
        if (consumer && s < Tb - 1) {
            const int snap = __builtin_amdgcn_readfirstlane(stage_p[s & 1][0]);
            if (snap > seen) seen = snap;
            if (rows_issued < s) {   // not requested yet: poll the producer's word
                int spins = 0;
                DAGX_STAMP(lane == 0, 5)   // (a step that had to poll)
                while (seen < s) {   // the rows of step s are published once the word reaches s
                    seen = __builtin_amdgcn_readfirstlane(load_agent(below));
                    if (seen >= s) break;
                    __builtin_amdgcn_s_sleep(2);
                    if (++spins > kSpinLimit) { s_abort = 1; break; }
                }
                if (seen >= s) { issue_rows(s, ln); wait_vmem_all(); }
            }
        }
        if (s + 1 < Tb) {
            issue_match(s + 1, ln);
            if (consumer && s + 1 < Tb - 1) {
                if (seen >= s + 1) issue_rows(s + 1, ln);
                dma_dword_agent(lds_addr(&stage_p[(s + 1) & 1][0]), below, 0u);
            }
        }
    };
    if (fetcher && Tb > 1) {   // what phase B of step 1 needs
        issue_match(1, lane);
        if (consumer && 1 < Tb - 1) dma_dword_agent(lds_addr(&stage_p[1][0]), below, 0u);
    }
    wait_vmem_all();
    __syncthreads();

    // What phase B needs for the block this wave owns (block jb0 + wave) does not change from step to step: its
    // first tile, its number of tiles and where its tile results lie.
    const bool own0 = wave < nblk;
    const int own_J = jb0 + wave, own_ilo = tile_ilo(own_J, W), own_nt = own_J - own_ilo + 1;
    auto part_row0 = [&](const int Jb) -> int {   // first result row of owned block Jb
        int row0 = 0;
        for (int J2 = jb0; J2 < Jb; ++J2) row0 += (J2 - tile_ilo(J2, W) + 1 + 7) & ~7;
        return row0;
    };
    const float *part_own = &part[own0 ? part_row0(own_J) : 0][lane];
    const int r16 = lane & 15;

    // the cell values of one owned block: maximum over its tiles (the first tile that attains it is remembered), plus
    // the match score; written to LDS for the next step and to the table
    auto finish_block = [&](const int Jb, const int ilo, const float best, const int from, const unsigned mraw, const int s, const int nxt,
                            const int lane) __attribute__((always_inline)) {
        const int p = Jb * kBlk + lane;
        const bool inband = p >= s && p <= slack + s;
        const float v = inband ? best + dma_decode<TM>(mraw) : DAGX_NEG_INF;   // second (and last) rounding of the cell
        abuf[nxt][Jb][lane] = v;
        if (p < Lb) { store_agent(cell(s, p), v); srcblk[s * spitch + p] = (unsigned char)(ilo + from); }
    };
    // maximum of eight tile results and the first place that holds it
    auto best_of_8 = [&](const float (&pv)[8], float &m, int &f) __attribute__((always_inline)) {
        m = max3(pv[0], pv[1], pv[2]);
        m = max3(m, pv[3], pv[4]);
        m = max3(m, pv[5], pv[6]);
        m = max3(m, pv[7], pv[7]);
        f = 7;
#pragma unroll
        for (int u = 6; u >= 0; --u) f = pv[u] == m ? u : f;
    };

    int cur = 0;
    for (int s = 1; s < Tb; ++s) {
        const int nxt = cur ^ 1;
        DAGX_STAMP(tid == 0, 1)
        // ---- phase A: tile max-plus products; the fetcher's copies ----
        if (__builtin_expect(fetcher, 0)) fetch_step(s);
        DAGX_STAMP(fetcher && lane == 0, 4)
        {
            // The scores for a tile are requested one tile ahead of its arithmetic.  A tile whose predecessor block
            // holds no finite score, or whose block lies outside the band, is skipped.
            float av[kTilesPerWave][4];
            bool geo[kTilesPerWave];
#define DAGX_ALIGN_READ(SL)                                                                        \
            geo[SL] = my_q[SL] >= 0 && my_J[SL] * kBlk <= slack + s && my_J[SL] * kBlk + kBlk - 1 >= s; \
            if (geo[SL]) {                                                                         \
                const float *ab = &abuf[cur][my_I[SL]][r16];                                       \
                av[SL][0] = ab[0]; av[SL][1] = ab[16]; av[SL][2] = ab[32]; av[SL][3] = ab[48];     \
            }
#define DAGX_ALIGN_TILE(SL, TILE)                                                                  \
            if (my_q[SL] >= 0) {                                                                   \
                float best = DAGX_NEG_INF;                                                         \
                if (geo[SL]) {                                                                     \
                    const float top = fmaxf(fmaxf(av[SL][0], av[SL][1]), fmaxf(av[SL][2], av[SL][3])); \
                    if (__builtin_amdgcn_ballot_w64(top > DAGX_NEG_INF) != 0)                     \
                        best = tile_maxplus(TILE, av[SL][0], av[SL][1], av[SL][2], av[SL][3]);     \
                }                                                                                  \
                part[my_q[SL]][lane] = best;                                                       \
            }
            DAGX_ALIGN_READ(0)
            DAGX_ALIGN_READ(1)
            DAGX_ALIGN_TILE(0, t0)
            DAGX_ALIGN_READ(2)
            DAGX_ALIGN_TILE(1, t1)
            DAGX_ALIGN_TILE(2, t2)
#undef DAGX_ALIGN_READ
#undef DAGX_ALIGN_TILE
        }
        // This wave's stores of step s-1 were issued in that step's phase B, a whole phase A ago: waiting for them
        // here costs nothing, and behind the barrier every wave has done so -- the progress word can say s-1 at the
        // start of phase B already, not at the end of the step.  (The fetcher's stores: it waited at the top of its
        // fetch; its requests for step s+1 stay in flight until the top of its next fetch.)
        if (!fetcher) wait_vmem_all();
        __syncthreads();
        DAGX_STAMP(tid == 0, 2)
        // ---- phase B ----
        if (__builtin_expect(tid == 0 && producer, 0)) store_agent(prog + g, s - 1);
        const int par = s & 1;
        const int gave_up_v = s_abort;   // set in phase A only; requested here, with the other LDS reads, and looked at behind the barrier
        if (own0) {
            const unsigned mraw = stage_m[par][wave][0][lane];
            float pv[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) pv[u] = part_own[u * kBlk];
            float best; int from;
            best_of_8(pv, best, from);
            if (!(best > DAGX_NEG_INF)) from = 0;
            for (int u0 = 8; u0 < own_nt; u0 += 8) {   // more than eight tiles: L > 512 with long links
#pragma unroll
                for (int u = 0; u < 8; ++u) pv[u] = part_own[(u0 + u) * kBlk];
                float m; int f;
                best_of_8(pv, m, f);
                if (m > best) { best = m; from = u0 + f; }
            }
            finish_block(own_J, own_ilo, best, from, mraw, s, nxt, lane);
        }
        for (int ob = wave + kTileWaves; ob < nblk; ob += kTileWaves) {   // a second owned block (narrow bands only)
            // (rare, so written to need few registers rather than to be fast: one tile result at a time,
            // and nothing of it computed ahead of the loop over the steps, where it would hold registers: hence 'ln')
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const int Jb = jb0 + ob, ilo = tile_ilo(Jb, W), nt = Jb - ilo + 1;
            const float *pr = &part[part_row0(Jb)][ln];
            const unsigned mraw = stage_m[par][wave][ob / kTileWaves][ln];
            float best = DAGX_NEG_INF;
            int from = 0;   // first tile (= lowest predecessor block) that attains the maximum
            for (int u = 0; u < nt; ++u) {
                const float x = pr[u * kBlk];
                if (x > best) { best = x; from = u; }
            }
            finish_block(Jb, ilo, best, from, mraw, s, nxt, ln);
        }
        if (consumer && s < Tb - 1) {
#pragma unroll
            for (int u = 0; u < kFetchSlots; ++u) {
                if (f_blk[u] < 0) continue;
                abuf[nxt][f_blk[u]][lane] = f_blk[u] * kBlk + lane < Lb ? stage_f[par][wave][u][lane] : DAGX_NEG_INF;
            }
        }
        __syncthreads();
        DAGX_STAMP(tid == 0, 3)
        if (__builtin_amdgcn_readfirstlane(gave_up_v)) {
            if (tid == 0) { a.flags[b] = 1; store_agent(prog + g, 1 << 30); }
            return;
        }
        cur = nxt;
    }
    if (producer) {
        wait_vmem_all();
        __syncthreads();
        if (tid == 0) store_agent(prog + g, Tb - 1);
    }
#undef DAGX_STAMP
}

// One wave per sample walks the path backwards through the score table.  The sweep has recorded, for
// every cell, the lowest block of 64 nodes that holds a best predecessor, so a step scans 64
// candidates (lanes <-> nodes of that block): it re-evaluates fl32(A[t-1][i] + E[i][j]) -- the very
// operation of the sweep, hence bit-identical -- takes the maximum and, among the lanes that hold it,
// the lowest node: the first-index rule of torch.max (fs_plugins/custom_ops/dag_loss.py:253-257, :350).
// The row of source blocks of step t-1 is fetched together with the candidates of step t (it does
// not depend on where the path goes), so a step costs one memory round trip.
//
// The workgroup has kOneGroupThreads threads all the same: a sample that the pipeline gave up on (flags[b] set) is
// done again here, from scratch, by the one-workgroup method; for every other sample all waves but the first leave
// at once.  (A launch of its own for the flagged samples, which are rare, would cost every call its latency.)
constexpr int kOneGroupThreads = 1024;
template <typename TM, typename TL, bool TRACE_LDS>
__global__ __launch_bounds__(kOneGroupThreads) void dag_backtrack_kernel(
    const float *__restrict__ table, const unsigned char *__restrict__ srcblk_all, const int *__restrict__ flags, AlignArgs a) {
    extern __shared__ float lds_a[];
    const int b = blockIdx.x;
    if (flags[b]) {
        align_one_sample<TM, TL, kOneGroupThreads, TRACE_LDS>(a, b, lds_a);
        return;
    }
    if (threadIdx.x >= kWave) return;
    const int lane = threadIdx.x;
    const int T = a.T, L = a.L, translen = a.translen;
    const int64_t *out_len = a.out_len, *tgt_len = a.tgt_len;
    const TL *links_all = static_cast<const TL *>(a.links);
    int64_t *path = a.path + (int64_t)b * L;
    for (int j = lane; j < L; j += kWave) path[j] = -1;
    const int Lb = (int)out_len[b], Tb = (int)tgt_len[b];
    if (!(Tb >= 1 && Lb >= 1 && Tb <= T && Lb <= L && Tb <= Lb)) return;
    const float *A = table + (int64_t)b * T * L;
    const int spitch = srcblk_pitch(L);
    const unsigned char *srcblk = srcblk_all + (int64_t)b * T * spitch;
    const TL *links = links_all + (int64_t)b * L * translen;
    if (!(A[(Tb - 1) * L + Lb - 1] > DAGX_NEG_INF)) return;   // no finite path
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");     // the -1 fill precedes the path entries (same wave)
    // a row of source blocks: L <= 1024 bytes, 16 per lane (lane l holds bytes 16 l .. 16 l + 15)
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    auto load_row = [&](int t, unsigned (&r)[4]) {   // rows are 16-byte aligned and padded to 16 bytes
        const u32x4 v = *reinterpret_cast<const u32x4 *>(srcblk + t * spitch + (16 * lane < spitch ? 16 * lane : 0));
        r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
    };
    unsigned row[4];
    if (Tb > 1) load_row(Tb - 1, row);
    int j = Lb - 1;
    for (int t = Tb - 1; t >= 1; --t) {
        if (lane == 0) path[j] = t;
        // source block of (t, j): byte j of the row
        const int q = (j >> 2) & 3, src_lane = j >> 4;
        const unsigned w = q == 0 ? row[0] : q == 1 ? row[1] : q == 2 ? row[2] : row[3];
        const int I = (int)((unsigned)__builtin_amdgcn_readlane((int)w, src_lane) >> (8 * (j & 3))) & 0xff;
        const int i = I * kBlk + lane;
        const int d = j - i - 1;
        const bool valid = d >= 0 && d < translen;
        const float e = to_float(links[valid ? i * translen + d : 0]);
        const float av = A[(t - 1) * L + (i < L ? i : L - 1)];
        if (t > 1) load_row(t - 1, row);                 // for the next step, in the same round trip
        const float x = valid ? av + e : DAGX_NEG_INF;
        const float top = wave64_max(x);
        if (!(top > DAGX_NEG_INF)) return;               // cannot happen on a finite path
        // lowest lane among those that hold the maximum
        j = I * kBlk + (int)__builtin_ctzll(__builtin_amdgcn_ballot_w64(x == top));
    }
    if (lane == 0) path[j] = 0;
}

constexpr size_t kAlignLdsBudget = 144 * 1024;


static bool trace_fits_lds(int T, int L) {
    return L <= 65535 && (size_t)L * 8 + (size_t)T * L * 2 <= kAlignLdsBudget;
}

// workspace: [score table B*T*L f32 | sync 16 + B*C ints | flags B ints | source blocks B*T*L bytes] (tile path) then
//            [trace B*T*L i32] when the back-pointers of the one-workgroup kernel do not fit LDS
static size_t align_tile_words(int B, int T, int L, int translen) {
    const int C = align_groups(B, L, translen);
    // the last terms: one byte per cell in rows of srcblk_pitch(L) bytes, and room to start them on a 16-byte boundary
    return C > 0 ? (size_t)B * T * L + 16 + (size_t)B * C + (size_t)B + 4 + (size_t)B * T * srcblk_pitch(L) / 4 : 0;
}
size_t align_workspace_bytes(int B, int T, int L, int translen) {
    return align_tile_words(B, T, L, translen) * 4 + (trace_fits_lds(T, L) ? 0 : (size_t)B * T * L * sizeof(int32_t));
}

// the pipeline words cleared; the flags of the samples ('nflags' words behind them) cleared too, or set (a test switch)
__global__ void dag_align_fill_kernel(int *p, int n, int nflags, int flag) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = i >= n - nflags ? flag : 0;
}

template <typename TM, typename TL>
static int launch_align(AlignArgs a, void *workspace, hipStream_t st) {
    constexpr int NT = 1024;
    const size_t tile_words = align_tile_words(a.B, a.T, a.L, a.translen);
    a.trace_ws = reinterpret_cast<int32_t *>(static_cast<float *>(workspace) + tile_words);
    int C = align_groups(a.B, a.L, a.translen);
    const int64_t span = (int64_t)(a.T - 1) * (a.ms1 < 0 ? -a.ms1 : a.ms1) + (int64_t)(a.L - 1) * (a.ms2 < 0 ? -a.ms2 : a.ms2);
    if (span >= (1LL << 31) / (int64_t)sizeof(TM) || a.ms1 < 0 || a.ms2 < 0 || force_log_domain()) C = 0;
    if (C > 0) {
        AlignTileArgs ta{};
        ta.match = a.match; ta.ms0 = a.ms0; ta.ms1 = a.ms1; ta.ms2 = a.ms2; ta.links = a.links;
        ta.out_len = a.out_len; ta.tgt_len = a.tgt_len; ta.B = a.B; ta.T = a.T; ta.L = a.L; ta.translen = a.translen;
        ta.table = static_cast<float *>(workspace);
        ta.sync = reinterpret_cast<int *>(ta.table + (size_t)a.B * a.T * a.L);
        ta.flags = ta.sync + 16 + a.B * C;
        ta.srcblk = reinterpret_cast<unsigned char *>((reinterpret_cast<uintptr_t>(ta.flags + a.B) + 15) & ~(uintptr_t)15);
        ta.C = C; ta.mcap = a.T - 1; ta.decode = 0;
        {
            const int W = (a.translen + kBlk - 1) / kBlk;
            int tmp[kTileCap + 2];
            for (int nb = 0; nb <= kMaxBlocksFast; ++nb) {
                partition_blocks(nb, W, C, tmp);
                for (int q = 0; q <= C && q < 12; ++q) ta.gtab[nb][q] = (unsigned char)tmp[q];
            }
        }
        const int nfill = 16 + a.B * C + a.B;
        hipLaunchKernelGGL(dag_align_fill_kernel, dim3((nfill + 255) / 256), dim3(256), 0, st, ta.sync, nfill, a.B, redo_every_sample() ? 1 : 0);
        int rc = check_launch("dag_align_fill");
        if (rc) return rc;
        const int B8 = (a.B + 7) & ~7;
        hipLaunchKernelGGL((dag_align_tiles_kernel<TM, TL>), dim3(B8 * C), dim3(kTileWaves * kWave), 0, st, ta);
        if ((rc = check_launch("dag_align_tiles"))) return rc;
        // the backtrack, and the samples that the pipeline gave up on
        const bool in_lds = trace_fits_lds(a.T, a.L);
        const size_t lds = (size_t)a.L * 8 + (in_lds ? (size_t)a.T * a.L * 2 : (size_t)0);
        auto kern = in_lds ? dag_backtrack_kernel<TM, TL, true> : dag_backtrack_kernel<TM, TL, false>;
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) { set_error("dag_best_alignment: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); return DAGX_ERR_LAUNCH; }
        }
        hipLaunchKernelGGL(kern, dim3(a.B), dim3(kOneGroupThreads), lds, st, ta.table, ta.srcblk, ta.flags, a);
        return check_launch("dag_backtrack");
    }
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
static int dispatch_align(int ldt, const AlignArgs &a, void *ws, hipStream_t st) {
    switch (ldt) {
        case DAGX_F32: return launch_align<TM, float>(a, ws, st);
        case DAGX_F16: return launch_align<TM, __half>(a, ws, st);
        default: return launch_align<TM, bf16_t>(a, ws, st);
    }
}

// ================================================================================================
// Viterbi decoding (fs_plugins/models/glat_decomposed_with_link.py:720-777)
// ================================================================================================
// The decoder's recursion  reach_t[j] = max_i fl32(reach_{t-1}[i] + E[i][j]) (+ u[j] in the joint
// form),  reach_0[j] = E[0][j] (+ u[0]) + u[j],  is the alignment sweep above with the table row
// s = t + 1, node 0 alone in row 0, and a three-row "match": row 0 = (u[0] or 0 at node 0), row 1 = u,
// rows >= 2 = (u or 0).  Every sample runs all `steps` = max_length + 1 rows and nothing is pruned
// towards the end, because a path may stop after any step: its score is reach_t[j] + E[j][L_b-1],
// divided by (t+1)^beta.  The sweep leaves the score table and the source blocks; one workgroup per
// sample then finds the best (t, j), walks back and collapses the tokens.
constexpr int kDecodeMaxSteps = 2049;   // max_length <= 2048 (= 2 L at L = 1024)
constexpr int kDecodeThreads = 1024;

// sync words <- 0, flags <- `flag`, match rows of every sample
__global__ void viterbi_prep_kernel(int *sync, int nsync, int *flags, int flag, const float *__restrict__ node_logp,
                                    int B, int L, int joint, float *__restrict__ match3) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < nsync) sync[i] = 0;
    if (i < B) flags[i] = flag;
    if (i < B * L) {
        const int b = i / L, j = i - b * L;
        const float u = node_logp[i];
        float *m = match3 + (int64_t)b * 3 * L;
        m[j] = (joint && j == 0) ? u : 0.0f;
        m[L + j] = u;
        m[2 * L + j] = joint ? u : 0.0f;
    }
}

// The table and the source blocks of one sample by one workgroup (a team of lanes <-> node, every lane scanning
// its predecessors in ascending order with a strict '>'): for the samples the pipeline did not do.
template <typename TL, int NT>
__global__ __launch_bounds__(NT) void viterbi_table_kernel(
    const float *__restrict__ match3, const TL *__restrict__ links_all, const int64_t *__restrict__ out_len,
    const int *__restrict__ flags, int T, int L, int translen, float *__restrict__ table_all,
    unsigned char *__restrict__ srcblk_all) {
    extern __shared__ float lds_v[];   // 2 L floats
    const int b = blockIdx.x, tid = threadIdx.x;
    if (!flags[b]) return;
    const int Lb = (int)out_len[b];
    if (!(Lb >= 1 && Lb <= L)) return;
    const float *m = match3 + (int64_t)b * 3 * L;
    const TL *links = links_all + (int64_t)b * L * translen;
    float *table = table_all + (int64_t)b * T * L;
    const int spitch = srcblk_pitch(L);
    unsigned char *srcblk = srcblk_all + (int64_t)b * T * spitch;
    float *fprev = lds_v, *fcur = lds_v + L;
    for (int j = tid; j < L; j += NT) {
        const float v = j == 0 ? m[0] : DAGX_NEG_INF;
        fprev[j] = v;
        if (j < Lb) table[j] = v;
    }
    __syncthreads();
    // a team of kTeam lanes <-> node, as in align_one_sample
    constexpr int kTeam = 8, R = 8;
    const int team = tid / kTeam, sub = tid % kTeam;
    const unsigned rs = (unsigned)(translen - 1);   // E[i][j-i-1] sits at links[i*(translen-1) + j-1]: 32-bit offsets
    for (int s = 1; s < T; ++s) {
        const float *mrow = m + (s < 2 ? s : 2) * L;
        for (int j = tid; j < Lb && j < s; j += NT) {   // not reachable in s steps
            fcur[j] = DAGX_NEG_INF;
            table[(int64_t)s * L + j] = DAGX_NEG_INF;
            srcblk[s * spitch + j] = 0;
        }
        for (int j = s + team; j < Lb; j += NT / kTeam) {
            const float mj = mrow[j];
            int ilo = j - translen; if (ilo < s - 1) ilo = s - 1;
            float best = DAGX_NEG_INF;
            int arg = ilo;
            const unsigned o_last = (unsigned)(j - 1) * (unsigned)translen;   // the offset of i = j-1, the largest
            unsigned o = (unsigned)(ilo + sub) * rs + (unsigned)(j - 1);
            for (int i0 = ilo + sub; i0 < j; i0 += kTeam * R, o += kTeam * R * rs) {
                float e[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const unsigned oc = o + (unsigned)(r * kTeam) * rs;
                    e[r] = to_float(links[oc < o_last ? oc : o_last]);
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const int i = i0 + r * kTeam;
                    const float x = i < j ? fprev[i < j ? i : j - 1] + e[r] : DAGX_NEG_INF;
                    if (x > best) { best = x; arg = i; }
                }
            }
#pragma unroll
            for (int w = kTeam / 2; w > 0; w >>= 1) {
                const float bo = __shfl_xor(best, w, kWave);
                const int ao = __shfl_xor(arg, w, kWave);
                if (bo > best || (bo == best && ao < arg)) { best = bo; arg = ao; }
            }
            if (sub == 0) {
                const float val = best + mj;
                fcur[j] = val;
                table[(int64_t)s * L + j] = val;
                srcblk[s * spitch + j] = (unsigned char)(arg / kBlk);
            }
        }
        __syncthreads();
        float *sw = fprev; fprev = fcur; fcur = sw;
    }
}

// the lowest index among the lanes whose value equals the wave's maximum; `top` receives that maximum
__device__ __forceinline__ int wave_first_argmax(float v, int idx, float &top) {
    top = wave64_max(v);
    const float cand = v == top ? (float)idx : 3.0e7f;   // indices < 2^24 are exact in float
    return (int)-wave64_max(-cand);
}

struct DecodeArgs {
    const float *table; const unsigned char *srcblk; const void *links;
    const int64_t *out_len, *node_tokens;
    const float *penalty;
    int T, L, translen, max_length;
    int64_t pad;
    int64_t *out_tokens, *out_count, *pred_length, *nodes;
};

template <typename TL>
__global__ __launch_bounds__(kDecodeThreads) void viterbi_select_kernel(DecodeArgs a) {
    __shared__ float sbest[kDecodeMaxSteps];
    __shared__ int sidx[kDecodeMaxSteps];
    __shared__ int walk[kDecodeMaxSteps];
    const int b = blockIdx.x, tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int L = a.L, T = a.T, translen = a.translen, n_max = a.max_length;
    const int Lb = (int)a.out_len[b];
    const float *A = a.table + (int64_t)b * T * L;
    const int spitch = srcblk_pitch(L);
    const unsigned char *srcblk = a.srcblk + (int64_t)b * T * spitch;
    const TL *links = static_cast<const TL *>(a.links) + (int64_t)b * L * translen;
    const int64_t *tok = a.node_tokens + (int64_t)b * L;
    int64_t *out_tokens = a.out_tokens + (int64_t)b * n_max;
    int64_t *nodes = a.nodes + (int64_t)b * n_max;
    const bool sane = Lb >= 1 && Lb <= L;

    // transition of every node to the last one: lane l holds nodes l, l + 64, ...
    float to_end[kMaxBlocksFast];
#pragma unroll
    for (int c = 0; c < kMaxBlocksFast; ++c) {
        const int j = c * kWave + lane, d = Lb - 1 - j - 1;
        const bool ok = sane && j < Lb && d >= 0 && d < translen;
        to_end[c] = ok ? to_float(links[(int64_t)j * translen + d]) : DAGX_NEG_INF;
    }
    // best node of every step (first index among equals, over all L nodes as the tensor formulation);
    // a wave takes kRows steps at a time so that their rows are in flight together
    constexpr int kRows = 4, kWaves = kDecodeThreads / kWave;
    const int nblk = (L + kWave - 1) / kWave;
    for (int t0 = wave * kRows; t0 < n_max; t0 += kWaves * kRows) {
        float best[kRows];
        int arg[kRows];
#pragma unroll
        for (int r = 0; r < kRows; ++r) { best[r] = DAGX_NEG_INF; arg[r] = lane; }
#pragma unroll
        for (int c = 0; c < kMaxBlocksFast; ++c) {
            if (c < nblk) {
                const int j = c * kWave + lane;
                float x[kRows];
#pragma unroll
                for (int r = 0; r < kRows; ++r) {
                    const int t = t0 + r < n_max ? t0 + r : n_max - 1;
                    x[r] = (sane && j < Lb) ? A[(int64_t)(t + 1) * L + j] : DAGX_NEG_INF;   // (j < Lb <= L)
                }
#pragma unroll
                for (int r = 0; r < kRows; ++r) {
                    const float v = x[r] + to_end[c];
                    if (v > best[r]) { best[r] = v; arg[r] = j; }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            float top;
            const int j0 = wave_first_argmax(best[r], arg[r], top);
            if (lane == 0 && t0 + r < n_max) { sbest[t0 + r] = top; sidx[t0 + r] = j0; }
        }
    }
    __syncthreads();
    if (wave != 0) return;
    // best length: score / (t+1)^beta, first index among equals
    float best = DAGX_NEG_INF;
    int arg = lane;
    for (int t = lane; t < n_max; t += kWave) {
        const float q = sbest[t] / a.penalty[t];
        if (q > best) { best = q; arg = t; }
    }
    float top;
    const int t_star = wave_first_argmax(best, arg, top);
    const int n = t_star + 1;
    int j = sidx[t_star];
    if (lane == 0) { a.pred_length[b] = n; walk[n - 1] = j; }
    // walk back: table row s = t + 1 holds reach_t; the predecessor of (s, j) lies in block srcblk[s][j]
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    auto load_row = [&](int s, unsigned (&r)[4]) {
        const u32x4 v = *reinterpret_cast<const u32x4 *>(srcblk + s * spitch + (16 * lane < spitch ? 16 * lane : 0));
        r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
    };
    unsigned rowb[4];
    if (n > 1) load_row(n, rowb);
    for (int s = n; s >= 2; --s) {
        const int q = (j >> 2) & 3, src_lane = j >> 4;
        const unsigned w = q == 0 ? rowb[0] : q == 1 ? rowb[1] : q == 2 ? rowb[2] : rowb[3];
        const int I = (int)((unsigned)__builtin_amdgcn_readlane((int)w, src_lane) >> (8 * (j & 3))) & 0xff;
        const int i = I * kBlk + lane;
        const int d = j - i - 1;
        const bool valid = d >= 0 && d < translen && i < L;
        const float e = to_float(links[valid ? (int64_t)i * translen + d : 0]);
        const float av = A[(int64_t)(s - 1) * L + (i < L ? i : L - 1)];
        if (s > 2) load_row(s - 1, rowb);
        const float x = valid ? av + e : DAGX_NEG_INF;
        float tp;
        const int lo = wave_first_argmax(x, lane, tp);
        j = tp > DAGX_NEG_INF ? I * kBlk + lo : 0;       // (a path of finite score never meets the other case)
        if (lane == 0) walk[s - 2] = j;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    // tokens: the last one always stays, an earlier one when it is not the pad and differs from its successor
    int count = 0;
    for (int k0 = 0; k0 < n_max; k0 += kWave) {
        const int k = k0 + lane;
        const bool in = k < n;
        const int node = in ? walk[k] : 0;
        const int64_t y = in ? tok[node] : a.pad;
        const int64_t ynext = (k + 1 < n) ? tok[walk[k + 1]] : a.pad;
        const bool keep = in && (k == n - 1 || (y != a.pad && y != ynext));
        const unsigned long long mask = __ballot(keep);
        const int pos = count + __popcll(mask & ((1ull << lane) - 1ull));
        if (keep) out_tokens[pos] = y;
        if (k < n_max) nodes[k] = in ? node : -1;
        count += __popcll(mask);
    }
    if (lane == 0) a.out_count[b] = count;
    for (int k = count + lane; k < n_max; k += kWave) out_tokens[k] = a.pad;
}

// workspace: [table B*T*L f32 | sync 16 + B*C | flags B | pad to 16 bytes | srcblk B*T*pitch bytes | match rows B*3*L f32]
static size_t decode_words(int B, int T, int L, int translen, int C) {
    return (size_t)B * T * L + 16 + (size_t)B * (C > 0 ? C : 1) + (size_t)B + 4 + (size_t)B * T * srcblk_pitch(L) / 4 + (size_t)B * 3 * L;
}
size_t decode_workspace_bytes(int B, int max_length, int L, int translen) {
    return decode_words(B, max_length + 1, L, translen, align_groups(B, L, translen)) * 4;
}

template <typename TL>
static int launch_decode(const void *links, const float *node_logp, const int64_t *node_tokens, const int64_t *out_len,
                         int B, int L, int translen, int max_length, const float *penalty, int joint, int64_t pad,
                         int64_t *out_tokens, int64_t *out_count, int64_t *pred_length, int64_t *nodes,
                         void *workspace, hipStream_t st) {
    const int T = max_length + 1;
    int C = align_groups(B, L, translen);
    const int Cw = C > 0 ? C : 1;
    if (force_log_domain()) C = 0;
    float *table = static_cast<float *>(workspace);
    int *sync = reinterpret_cast<int *>(table + (size_t)B * T * L);
    int *flags = sync + 16 + B * Cw;
    unsigned char *srcblk = reinterpret_cast<unsigned char *>((reinterpret_cast<uintptr_t>(flags + B) + 15) & ~(uintptr_t)15);
    float *match3 = reinterpret_cast<float *>(srcblk + (size_t)B * T * srcblk_pitch(L));
    const int nsync = 16 + B * Cw;
    const int nprep = B * L > nsync ? B * L : nsync;
    hipLaunchKernelGGL(viterbi_prep_kernel, dim3((nprep + 255) / 256), dim3(256), 0, st, sync, nsync, flags, C > 0 ? 0 : 1,
                       node_logp, B, L, joint, match3);
    int rc = check_launch("viterbi_prep");
    if (rc) return rc;
    if (C > 0) {
        AlignTileArgs ta{};
        ta.match = match3; ta.ms0 = 3 * (int64_t)L; ta.ms1 = L; ta.ms2 = 1; ta.links = links;
        ta.out_len = out_len; ta.tgt_len = nullptr; ta.B = B; ta.T = T; ta.L = L; ta.translen = translen;
        ta.table = table; ta.sync = sync; ta.flags = flags; ta.srcblk = srcblk;
        ta.C = C; ta.mcap = 2; ta.decode = 1;
        const int W = (translen + kBlk - 1) / kBlk;
        int tmp[kTileCap + 2];
        for (int nb = 0; nb <= kMaxBlocksFast; ++nb) {
            partition_blocks(nb, W, C, tmp);
            for (int q = 0; q <= C && q < 12; ++q) ta.gtab[nb][q] = (unsigned char)tmp[q];
        }
        const int B8 = (B + 7) & ~7;
        hipLaunchKernelGGL((dag_align_tiles_kernel<float, TL>), dim3(B8 * C), dim3(kTileWaves * kWave), 0, st, ta);
        if ((rc = check_launch("viterbi_tiles"))) return rc;
    }
    constexpr int NT = 1024;
    hipLaunchKernelGGL((viterbi_table_kernel<TL, NT>), dim3(B), dim3(NT), (size_t)L * 8, st, match3, static_cast<const TL *>(links),
                       out_len, flags, T, L, translen, table, srcblk);
    if ((rc = check_launch("viterbi_table"))) return rc;
    DecodeArgs d{table, srcblk, links, out_len, node_tokens, penalty, T, L, translen, max_length, pad,
                 out_tokens, out_count, pred_length, nodes};
    hipLaunchKernelGGL((viterbi_select_kernel<TL>), dim3(B), dim3(kDecodeThreads), 0, st, d);
    return check_launch("viterbi_select");
}

}  // namespace dagx

using namespace dagx;

extern "C" int dagx_best_alignment(const void *match, int match_dtype, const int64_t match_strides[3],
                                   const void *links, int links_dtype,
                                   const int64_t *out_len, const int64_t *tgt_len,
                                   int B, int T, int L, int translen,
                                   int64_t *path, void *workspace, size_t workspace_bytes, void *stream) {
    if (B < 0 || T < 1 || L < 1 || translen < 1) { set_error("dag_best_alignment: bad sizes B=%d T=%d L=%d translen=%d", B, T, L, translen); return DAGX_ERR_ARGUMENT; }
    if (B == 0) return DAGX_OK;                 // an empty batch owns no memory: nothing to check or launch
    if (!match || !match_strides || !links || !out_len || !tgt_len || !path) { set_error("dag_best_alignment: null pointer argument"); return DAGX_ERR_ARGUMENT; }
    if (match_dtype < DAGX_F32 || match_dtype > DAGX_BF16 || links_dtype < DAGX_F32 || links_dtype > DAGX_BF16) { set_error("dag_best_alignment: unsupported dtype"); return DAGX_ERR_ARGUMENT; }
    if (L > 8192) { set_error("dag_best_alignment: graph size L=%d exceeds the supported 8192", L); return DAGX_ERR_UNSUPPORTED; }
    size_t need = align_workspace_bytes(B, T, L, translen);
    if (need > 0 && (!workspace || workspace_bytes < need)) { set_error("dag_best_alignment: workspace of %zu bytes required, %zu given", need, workspace_bytes); return DAGX_ERR_WORKSPACE; }
    AlignArgs a{match, match_strides[0], match_strides[1], match_strides[2], links, out_len, tgt_len,
                B, T, L, translen, path, nullptr};
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (match_dtype) {
        case DAGX_F32: return dispatch_align<float>(links_dtype, a, workspace, st);
        case DAGX_F16: return dispatch_align<__half>(links_dtype, a, workspace, st);
        default: return dispatch_align<bf16_t>(links_dtype, a, workspace, st);
    }
}

extern "C" int dagx_viterbi_decode(const void *links, int links_dtype, const float *node_logp, const int64_t *node_tokens,
                                   const int64_t *out_len, int B, int L, int translen, int max_length,
                                   const float *length_penalty, int joint, int64_t pad,
                                   int64_t *out_tokens, int64_t *out_count, int64_t *pred_length, int64_t *nodes,
                                   void *workspace, size_t workspace_bytes, void *stream) {
    if (B < 0 || L < 1 || translen < 1 || max_length < 1) { set_error("dag_viterbi_decode: bad sizes B=%d L=%d translen=%d max_length=%d", B, L, translen, max_length); return DAGX_ERR_ARGUMENT; }
    if (B == 0) return DAGX_OK;
    if (!links || !node_logp || !node_tokens || !out_len || !length_penalty || !out_tokens || !out_count || !pred_length || !nodes) { set_error("dag_viterbi_decode: null pointer argument"); return DAGX_ERR_ARGUMENT; }
    if (links_dtype < DAGX_F32 || links_dtype > DAGX_BF16) { set_error("dag_viterbi_decode: unsupported dtype"); return DAGX_ERR_ARGUMENT; }
    if (L > kMaxBlocksFast * kBlk) { set_error("dag_viterbi_decode: graph size L=%d exceeds the supported %d", L, kMaxBlocksFast * kBlk); return DAGX_ERR_UNSUPPORTED; }
    if (max_length + 1 > kDecodeMaxSteps) { set_error("dag_viterbi_decode: max_length=%d exceeds the supported %d", max_length, kDecodeMaxSteps - 1); return DAGX_ERR_UNSUPPORTED; }
    if ((int64_t)B * (max_length + 1) * L > 0x7fffffffLL) { set_error("dag_viterbi_decode: B*(max_length+1)*L too large for one call"); return DAGX_ERR_UNSUPPORTED; }
    const size_t need = decode_workspace_bytes(B, max_length, L, translen);
    if (!workspace || workspace_bytes < need) { set_error("dag_viterbi_decode: workspace of %zu bytes required, %zu given", need, workspace_bytes); return DAGX_ERR_WORKSPACE; }
    hipStream_t st = static_cast<hipStream_t>(stream);
#define DAGX_GO(TL) launch_decode<TL>(links, node_logp, node_tokens, out_len, B, L, translen, max_length, length_penalty, joint, pad, \
                                      out_tokens, out_count, pred_length, nodes, workspace, st)
    switch (links_dtype) {
        case DAGX_F32: return DAGX_GO(float);
        case DAGX_F16: return DAGX_GO(__half);
        default: return DAGX_GO(bf16_t);
    }
#undef DAGX_GO
}

extern "C" size_t dagx_workspace_bytes(int op, int B, int T, int L, int translen) {
    if (B <= 0 || T <= 0 || L <= 0) return 0;
    if (op == DAGX_OP_VITERBI_DECODE) return L <= kMaxBlocksFast * kBlk ? decode_workspace_bytes(B, T, L, translen) : 0;
    if (op == DAGX_OP_BEST_ALIGNMENT) return align_workspace_bytes(B, T, L, translen);
    if (op == DAGX_OP_BEST_ALIGNMENT_F64) return align_f64_workspace_bytes(B, T, L);
    if (op == DAGX_OP_LOSS_FWD) return loss_fwd_workspace_bytes(B, T, L, translen);
    if (op == DAGX_OP_LOSS_BWD) return loss_bwd_workspace_bytes(B);
    return 0;
}

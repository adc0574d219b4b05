// Building blocks shared by the tile-resident sweep kernels (log-semiring loss, max-semiring
// alignment): tile geometry, the grouping of position blocks into a pipeline of workgroups, DPP
// broadcast arithmetic and lane reductions, agent-scope loads/stores for the hand-over.
#pragma once

#include "dagx_common.h"

namespace dagx {

constexpr int kBlk = 64;            // positions per block
constexpr int kMaxBlocksFast = 16;  // fast path: L <= 1024
constexpr int kTileWaves = 8;       // waves per workgroup in the fast sweep
constexpr int kTilesPerWave = 3;    // register-resident tiles per wave
constexpr int kTileCap = kTileWaves * kTilesPerWave;
// Linear-domain numbers of the fast sweep carry a constant factor 2^kShift2 each (transition probabilities
// and exp(residual) alike), so that the fp32 exponent range is used on both sides of 1: a transition or a
// residual survives down to exp(-126) instead of exp(-87), their product down to exp(-165).  Sums of
// products stay below 2^(2 * 56 + 10) < 2^128.
constexpr int kShift2 = 56;                       // in log2 units (38.8 nats)
constexpr float kMinLogP = -87.0f - 38.8f;        // a finite transition below this has no normal number in the scaled linear domain
constexpr float kTinyStored = 1.17549435e-38f;    // 2^-126: the smallest number that domain holds (a factor of exp(-126) under its scale)
constexpr int kSpinLimit = 1 << 22;

struct Tile { float p[kBlk]; };

// acc += sum_{r<16} e[lane r of this lane's 16-lane row] * p[r]
__device__ __forceinline__ void fma16_rowbcast(float &acc, float e, const float *p) {
    asm(
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %1, %2 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %3 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %4 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %5 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %6 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %7 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %8 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %9 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %10 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %11 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %12 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %13 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %14 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %15 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %16 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %17 row_newbcast:15 row_mask:0xf bank_mask:0xf"
        : "+v"(acc)
        : "v"(e), "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]),
          "v"(p[8]), "v"(p[9]), "v"(p[10]), "v"(p[11]), "v"(p[12]), "v"(p[13]), "v"(p[14]), "v"(p[15]));
}

// acc = sum_{r<16} e[lane r of this lane's 16-lane row] * p[r]  (starts the sum: no zeroed accumulator needed)
__device__ __forceinline__ void mul16_rowbcast(float &acc, float e, const float *p) {
    asm(
        "s_nop 1\n\t"
        "v_mul_f32_dpp %0, %1, %2 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %3 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %4 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %5 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %6 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %7 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %8 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %9 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %10 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %11 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %12 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %13 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %14 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %15 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %16 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
        "v_fmac_f32_dpp %0, %1, %17 row_newbcast:15 row_mask:0xf bank_mask:0xf"
        : "=&v"(acc)
        : "v"(e), "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]),
          "v"(p[8]), "v"(p[9]), "v"(p[10]), "v"(p[11]), "v"(p[12]), "v"(p[13]), "v"(p[14]), "v"(p[15]));
}

// acc (+)= sum_{u<4} f[lane U0+u of this lane's 16-lane row] * v[u]: four values per lane, each scaled by a factor
// that sits in one lane of a 16-replicated vector.  U0 = 0 starts the sum with a multiply.  (Four at a time: with
// eight operands per statement the register allocator had to evict tile registers around it.)
template <int U0>
__device__ __forceinline__ void scaled_sum4(float &acc, float f, float v0, float v1, float v2, float v3) {
    static_assert(U0 % 4 == 0 && U0 >= 0 && U0 < 16, "");
    if constexpr (U0 == 0) {
        asm("s_nop 1\n\t"
            "v_mul_f32_dpp %0, %1, %2 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %1, %3 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %1, %4 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %1, %5 row_newbcast:3 row_mask:0xf bank_mask:0xf"
            : "=&v"(acc) : "v"(f), "v"(v0), "v"(v1), "v"(v2), "v"(v3));
    } else {
        asm("s_nop 1\n\t"
            "v_fmac_f32_dpp %0, %1, %2 row_newbcast:%c6 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %1, %3 row_newbcast:%c7 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %1, %4 row_newbcast:%c8 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32_dpp %0, %1, %5 row_newbcast:%c9 row_mask:0xf bank_mask:0xf"
            : "+v"(acc) : "v"(f), "v"(v0), "v"(v1), "v"(v2), "v"(v3), "n"(U0), "n"(U0 + 1), "n"(U0 + 2), "n"(U0 + 3));
    }
}

// Number of tiles of position block Jb: predecessor blocks I in [ilo, Jb]; W = blocks a transition can span.
__device__ __host__ __forceinline__ int tile_ilo(int Jb, int W) { return Jb > W ? Jb - W : 0; }

// Contiguous grouping of the position blocks [0, NBb) into at most C groups of at most kTileCap tiles,
// minimising the largest group.  gstart[g] .. gstart[g+1] are the blocks of group g (empty groups last).
__device__ __host__ inline int partition_blocks(int NBb, int W, int C, int *gstart) {
    int best_cap = kTileCap;
    for (int cap = 1; cap <= kTileCap; ++cap) {
        int groups = 1, sum = 0; bool ok = true;
        for (int Jb = 0; Jb < NBb; ++Jb) {
            int c = Jb - tile_ilo(Jb, W) + 1;
            if (c > cap) { ok = false; break; }
            if (sum + c > cap) { ++groups; sum = 0; }
            sum += c;
        }
        if (ok && groups <= C) { best_cap = cap; break; }
    }
    int g = 0, sum = 0;
    gstart[0] = 0;
    for (int Jb = 0; Jb < NBb; ++Jb) {
        int c = Jb - tile_ilo(Jb, W) + 1;
        if (sum + c > best_cap && sum > 0) { ++g; if (g < C) gstart[g] = Jb; sum = 0; }
        sum += c;
    }
    int used = g + 1;
    for (int q = used; q <= C; ++q) gstart[q] = NBb;
    return used;
}

// Host: workgroups per sweep needed for graph size L (0 = the fast path does not apply).
inline int groups_needed(int L, int translen) {
    const int NB = (L + kBlk - 1) / kBlk;
    if (NB > kMaxBlocksFast) return 0;
    const int W = (translen + kBlk - 1) / kBlk;
    int groups = 1, sum = 0;
    for (int Jb = 0; Jb < NB; ++Jb) {
        int c = Jb - tile_ilo(Jb, W) + 1;
        if (c > kTileCap) return 0;
        if (sum + c > kTileCap) { ++groups; sum = 0; }
        sum += c;
    }
    return groups <= 11 ? groups : 0;
}

// Host: workgroups per sweep actually launched.  More groups than needed mean fewer tiles per SIMD but a
// hand-over between groups in every step and a deeper pipeline.  Measured on MI355X (B = 16..64, T = 64):
// the loss sweeps (two per sample, a heavier owner phase) are fastest with the minimal number at every
// graph size but 384 (there 6 % slower than with twice as many; at 128 and 256 nodes 20-26 % faster); the
// alignment sweep gains 5-13 % from doubling the groups once when the graph has at least 4 blocks and the
// device has room (one workgroup per CU), and loses from doubling twice; where twice the minimal number
// exceeds the 11 the kernel supports (L > 704), 10 groups are used when they fit.
inline int groups_used(int sweeps, int L, int translen, bool may_double) {
    int C = groups_needed(L, translen);
    if (C == 0) return 0;
    const int NB = (L + kBlk - 1) / kBlk;
    if (may_double) {
        if (NB >= 4 && 2 * C <= 11 && 2 * C <= NB && (long long)sweeps * 2 * C <= 256) C *= 2;
        else if (C < 10 && NB >= 10 && (long long)sweeps * 10 <= 256) C = 10;   // L=1024, T=256, B=16: 0.93 -> 0.82 ms
    }
    return C;
}

// ---- DPP lane reductions (no LDS traffic) ----------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v),
                                                                 CTRL, 0xf, 0xf, false));
}
// max over each 16-lane row, result in every lane of the row (butterfly; each DPP op needs its
// source written two wait states earlier)
__device__ __forceinline__ float row16_max(float v) {
    float r;
    asm("s_nop 1\n\t"
        "v_max_f32_dpp %0, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf"
        : "=&v"(r) : "v"(v));
    return r;
}
// inclusive prefix max within each 16-lane row: lane k gets max over lanes 0..k of the row
__device__ __forceinline__ float row16_prefix_max(float v) {
    asm("s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_shr:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_shr:8 row_mask:0xf bank_mask:0xf"
        : "+v"(v));
    return v;
}
__device__ __forceinline__ float lane_bcast(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
// max over the 64 lanes, wave-uniform result: butterfly inside the 16-lane rows, then the row
// results are folded across rows with the two wave-level DPP broadcasts (row 0 -> 1, row 2 -> 3 via
// row_bcast:15; rows 0-1 -> rows 2-3 via row_bcast:31) and lane 63 holds the maximum.
__device__ __forceinline__ float wave64_max(float v) {
    v = row16_max(v);
    asm("s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf"
        : "+v"(v));
    return lane_bcast(v, 63);
}

// A wave-uniform value the compiler must take as new at this point: address arithmetic built on it
// stays inside the loop (as one add per use) instead of being hoisted into a vector register that
// then lives across the whole loop.
__device__ __forceinline__ int opaque_uniform(int x) { asm volatile("" : "+s"(x)); return x; }

template <typename X>
__device__ __forceinline__ X load_agent(const X *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
template <typename X>
__device__ __forceinline__ void store_agent(X *p, X v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Wait until every vector-memory operation of this wave has completed.  Written as the builtin, not as
// inline assembly: the compiler's own wait-count bookkeeping then knows that nothing is outstanding and
// adds no second wait (which would also cover the stores issued in between) where a loop-carried load
// destination is rewritten.  Encoding: vmcnt = 0, expcnt = 7 (no wait), lgkmcnt = 15 (no wait).
// The empty asm statements keep the compiler from moving memory operations across the wait.
__device__ __forceinline__ void wait_vmem_all() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" ::: "memory");
}

// Asynchronous copy global -> LDS, one element per lane ("LDS-direct" load): the element at
// gbase + voff (bytes, per lane) lands in the dword at LDS byte address lds_byte + 4 * lane (16-bit
// elements zero-extended).  The hardware counts it in vmcnt like any vector load and completes it in
// issue order with the other vector loads and stores of the wave, but the compiler's wait-count
// bookkeeping does not see it: the code that uses these must place its own s_waitcnt (wait_vmem_*)
// before the data is read, and must not rely on compiler-computed vmcnt(N > 0) waits for other loads
// while such copies are in flight.
// the address as a value the compiler knows to be wave-uniform (so that it is handed to the
// instruction in scalar registers)
__device__ __forceinline__ unsigned long long uniform_address(const void *p) {
    const unsigned long long v = reinterpret_cast<unsigned long long>(p);
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(v & 0xffffffffULL));
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(v >> 32));
    return ((unsigned long long)hi << 32) | lo;
}
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma_dword(unsigned lds_byte, const void *gbase, unsigned voff) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" :: "v"(voff), "s"(uniform_address(gbase)), "s"(lds_byte) : "memory", "m0");
}
__device__ __forceinline__ void dma_dword_agent(unsigned lds_byte, const void *gbase, unsigned voff) {   // agent-scope (sc1) load
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1 sc1" :: "v"(voff), "s"(uniform_address(gbase)), "s"(lds_byte) : "memory", "m0");
}
__device__ __forceinline__ void dma_ushort(unsigned lds_byte, const void *gbase, unsigned voff) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_ushort %0, %1" :: "v"(voff), "s"(uniform_address(gbase)), "s"(lds_byte) : "memory", "m0");
}
// The same with the base address already in scalar registers (a value taken through uniform_address once).
__device__ __forceinline__ void dma_dword_u(unsigned lds_byte, unsigned long long ubase, unsigned voff) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" :: "v"(voff), "s"(ubase), "s"(lds_byte) : "memory", "m0");
}
__device__ __forceinline__ void dma_dword_agent_u(unsigned lds_byte, unsigned long long ubase, unsigned voff) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1 sc1" :: "v"(voff), "s"(ubase), "s"(lds_byte) : "memory", "m0");
}
__device__ __forceinline__ void dma_ushort_u(unsigned lds_byte, unsigned long long ubase, unsigned voff) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_ushort %0, %1" :: "v"(voff), "s"(ubase), "s"(lds_byte) : "memory", "m0");
}
#pragma clang diagnostic pop
template <typename X> __device__ __forceinline__ void dma_elem_u(unsigned lds_byte, unsigned long long ubase, unsigned voff) {
    if constexpr (sizeof(X) == 4) dma_dword_u(lds_byte, ubase, voff); else dma_ushort_u(lds_byte, ubase, voff);
}
template <typename X> __device__ __forceinline__ void dma_elem(unsigned lds_byte, const X *gbase, unsigned voff);
template <> __device__ __forceinline__ void dma_elem<float>(unsigned lds_byte, const float *gbase, unsigned voff) { dma_dword(lds_byte, gbase, voff); }
template <> __device__ __forceinline__ void dma_elem<__half>(unsigned lds_byte, const __half *gbase, unsigned voff) { dma_ushort(lds_byte, gbase, voff); }
template <> __device__ __forceinline__ void dma_elem<bf16_t>(unsigned lds_byte, const bf16_t *gbase, unsigned voff) { dma_ushort(lds_byte, gbase, voff); }
// value of an element that dma_elem<X> left in an LDS dword
template <typename X> __device__ __forceinline__ float dma_decode(unsigned raw);
template <> __device__ __forceinline__ float dma_decode<float>(unsigned raw) { return __builtin_bit_cast(float, raw); }
template <> __device__ __forceinline__ float dma_decode<__half>(unsigned raw) { return __half2float(__builtin_bit_cast(__half, (unsigned short)raw)); }
template <> __device__ __forceinline__ float dma_decode<bf16_t>(unsigned raw) { return __builtin_bit_cast(float, raw << 16); }

// Wait until at most `pending` (0..6) of this wave's vector-memory operations are outstanding (they
// complete in issue order, so the oldest ones are done).
__device__ __forceinline__ void wait_vmem_but(int pending) {
    asm volatile("" ::: "memory");
    switch (pending) {
        case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
        case 1: __builtin_amdgcn_s_waitcnt(0x0F71); break;
        case 2: __builtin_amdgcn_s_waitcnt(0x0F72); break;
        case 3: __builtin_amdgcn_s_waitcnt(0x0F73); break;
        case 4: __builtin_amdgcn_s_waitcnt(0x0F74); break;
        case 5: __builtin_amdgcn_s_waitcnt(0x0F75); break;
        default: __builtin_amdgcn_s_waitcnt(0x0F76); break;
    }
    asm volatile("" ::: "memory");
}

// Stage one tile: t.p[r] = exp(E(pred position 64*I + r -> position 64*Jb + lane)), 0 where there is
// no such transition (EXP), or the log value itself, -inf where there is none (!EXP).  In the shifted layout the element sits at row*translen + d with
// d = p_out - p_in - 1.
//  * alpha (row = p_in): for a fixed r the 64 lanes read 64 consecutive elements -> coalesced as is.
//  * beta (row = L_b-1-p_out): a lane's 64 values are consecutive in memory, the lanes are a whole
//    row apart.  The wave therefore reads row by row (lanes <-> r, coalesced) and transposes
//    through a private LDS patch.
// Loads are unconditional (clamped to element 0) so that all 64 of a tile can be in flight.
// 2^(x + kShift2) and log2(y) - 2 * kShift2 with the rounding errors of the unshifted functions: the shift goes
// through the exponent field (ldexp / frexp), not through the argument of v_exp_f32 or the result of
// v_log_f32, where adding 56 would cost five bits of the fraction.
__device__ __forceinline__ float exp2_shifted(float x) {
    // (arguments below -115, results under 2^-59, take the shift inside the argument instead: v_exp_f32 alone
    //  would flush them, and their rounding no longer matters)
    const bool deep = x < -115.f;
    const float r = fast_exp2(deep ? x + (float)kShift2 : x);
    return deep ? r : __builtin_ldexpf(r, kShift2);
}
// The staged transitions of the wide (float64) sweeps carry 2^kShiftLinksWide instead: their products are formed
// in float64, so the whole range of normal float32 numbers lies under a transition of probability one --
// log-probabilities down to kMinLogPWide = -(126 + 127) ln 2, rounded up.  (Not the subnormals below it: a
// subnormal has lost bits of its fraction, a transition of -190 came out 8 % off, and both sweeps of a sample
// carried the same wrong number, so nothing flagged it.  A log-probability above 0 overflows; the sample then
// fails its check and goes to the log-domain kernel.)
constexpr int kShiftLinksWide = 127;
constexpr float kMinLogPWide = -175.0f;
template <int SHIFT>
__device__ __forceinline__ float exp2_shifted_by(float x) {
    if constexpr (SHIFT == kShift2) return exp2_shifted(x);
    const bool deep = x < -115.f;   // (through a lifted argument, so that v_exp_f32 has a normal result, and down again by ldexp, which keeps subnormals)
    const float r = fast_exp2(deep ? x + (float)(SHIFT + 24) : x);
    return __builtin_ldexpf(r, deep ? -24 : SHIFT);
}
template <int SHIFT> __device__ __forceinline__ constexpr float min_logp() { return SHIFT == kShift2 ? kMinLogP : kMinLogPWide; }
__device__ __forceinline__ float log2_unshifted(float y) {   // y > 0
    return (float)(__builtin_amdgcn_frexp_expf(y) - 2 * kShift2) + fast_log2(__builtin_amdgcn_frexp_mantf(y));
}

// `tiny`: what a finite transition too small for the linear domain becomes -- 0 in a sweep that must never
// overstate (a lower bound of every sum), kTinyStored in one that must never understate (an upper bound).
template <bool EXP, int SHIFT>
__device__ __forceinline__ float link_prob(float e, bool valid, float tiny) {
    if (EXP) {   // linear domain (scaled by 2^SHIFT); a NaN stays a NaN, as in the short forms below
        if (!valid) return 0.f;
        if (e <= min_logp<SHIFT>()) return e > DAGX_NEG_INF ? tiny : 0.f;
        return exp2_shifted_by<SHIFT>(e * kLog2e);
    }
    return valid ? e : DAGX_NEG_INF;                                           // log domain as is
}

// The staging is bound by vector-instruction issue, not by memory (the same loads alone run at 6 TB/s): with the
// validity tests, the test for tiny values and the two-branch exponential an element costs 16 instructions.  A tile
// whose 64 x 64 positions are all transitions (most tiles: not on the diagonal, not at the end of the sample or of
// the band) needs none of the tests, and a value needs the long form of the exponential only below -79.  So a batch
// of such a tile first looks for the most negative finite value each lane has loaded (two instructions per element),
// and unless some lane has one below -79 it is converted the short way: scale, exp, ldexp.  A batch of any other tile
// (on the diagonal, at the end of the sample or of the band) does the same over its valid elements and then puts 0 in
// the places that are no transitions: 9 instructions.  Only a batch with a value below -79 takes the long way.  Same
// values either way.
//
// `lowest` tracks 0xff7fffff - bits(e): smallest for the most negative finite e (positive values, -inf and NaNs come
// out large).
// (Taken from the element as it was loaded: a half needs no conversion for this, and its conversion then folds
//  into the scaling, v_fma_mix_f32.)
__device__ __forceinline__ unsigned lowest_key(float e) { return 0xff7fffffu - __builtin_bit_cast(unsigned, e); }
__device__ __forceinline__ unsigned lowest_key(__half e) { return 0xfbffu - (unsigned)__builtin_bit_cast(unsigned short, e); }
__device__ __forceinline__ unsigned lowest_key(bf16_t e) { return 0xff7fu - (unsigned)e.bits; }
// lowest_key < this: some finite e < -79
__device__ __forceinline__ constexpr unsigned lowest_deep(float) { return 0xff7fffffu - 0xc29e0000u; }
__device__ __forceinline__ constexpr unsigned lowest_deep(__half) { return 0xfbffu - 0xd4f0u; }
__device__ __forceinline__ constexpr unsigned lowest_deep(bf16_t) { return 0xff7fu - 0xc29eu; }
template <int CH, typename TL>
__device__ __forceinline__ bool batch_is_plain(const TL (&e)[CH]) {
    unsigned lowest = 0xffffffffu;
#pragma unroll
    for (int r = 0; r < CH; ++r) {
        const unsigned u = lowest_key(e[r]);
        lowest = u < lowest ? u : lowest;
    }
    return __builtin_amdgcn_ballot_w64(lowest < lowest_deep(TL{})) == 0;
}
template <int CH, typename TL>
__device__ __forceinline__ bool batch_is_plain(const TL (&e)[CH], const bool (&valid)[CH]) {
    unsigned lowest = 0xffffffffu;
#pragma unroll
    for (int r = 0; r < CH; ++r) {
        const unsigned u = valid[r] ? lowest_key(e[r]) : 0xffffffffu;
        lowest = u < lowest ? u : lowest;
    }
    return __builtin_amdgcn_ballot_w64(lowest < lowest_deep(TL{})) == 0;
}
// e * log2(e) as link_prob computes it (a product with a zero added rounds like the product)
__device__ __forceinline__ float times_log2e(float e) { return e * kLog2e; }
__device__ __forceinline__ float times_log2e(__half e) { return __builtin_fmaf(__half2float(e), kLog2e, 0.0f); }
__device__ __forceinline__ float times_log2e(bf16_t e) { return to_float(e) * kLog2e; }
template <bool EXP, int SHIFT, typename TL>
__device__ __forceinline__ float plain_value(TL e) {   // link_prob for a valid element that is -inf or >= -79
    if (EXP) return __builtin_ldexpf(fast_exp2(times_log2e(e)), SHIFT);
    return to_float(e);
}

template <bool EXP, int CH, typename TL, int SHIFT = kShift2>
__device__ __forceinline__ void load_tile(Tile &t, const TL *links, int I, int Jb, int lane, int dir, int Lb, int translen,
                                          float (*stage)[kBlk + 1], float tiny) {
    const int dd = (Jb - I) * kBlk - 1;   // d = dd + (lane of p_out) - r
    // CH loads are in flight per batch.  An address is the sample's (uniform) base plus a 32-bit byte offset per lane:
    // one register per load in flight, which the loaded value then takes over.  Measured: the loss sweeps (both
    // directions staging at once) are fastest with 16 (32 costs the beta staging 4 us, 64 everything 8 us); the
    // alignment sweep, which stages fp32 tiles in one direction only, gains from 32 (-2 us at L=512, -5 % at L=1024).
    const char *const lbase = reinterpret_cast<const char *>(links);
    auto at = [&](const bool valid, const int index) __attribute__((always_inline)) -> TL {
        return *reinterpret_cast<const TL *>(lbase + (valid ? (unsigned)index * (unsigned)sizeof(TL) : 0u));
    };
    // every (row, lane) of the tile is a transition of the sample (wave-uniform)
    const bool interior = Jb > I && dd + kBlk - 1 < translen && Jb * kBlk + kBlk - 1 < Lb;
    // The loads of a batch are requested before the batch in front of it is converted (two batches of registers),
    // so that the conversion arithmetic runs under the memory time of the next loads.
    constexpr int NB = kBlk / CH;
    if (dir == 0) {
        const int p_out = Jb * kBlk + lane;
        const int base = I * kBlk * translen + dd + lane;
        const int step = translen - 1;
        const bool col_ok = p_out < Lb;
        TL raw[2][CH];
        auto request = [&](const int c, TL (&dst)[CH]) __attribute__((always_inline)) {
#pragma unroll
            for (int r = 0; r < CH; ++r) {
                const int d = dd + lane - (c + r);
                const bool valid = col_ok && d >= 0 && d < translen;
                dst[r] = at(interior || valid, base + (c + r) * step);
            }
        };
        request(0, raw[0]);
#pragma unroll
        for (int k = 0; k < NB; ++k) {
            const int c = k * CH;
            if (k + 1 < NB) request(c + CH, raw[(k + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            const TL (&e)[CH] = raw[k & 1];
            if (interior) {
                if (!EXP || batch_is_plain<CH>(e)) {
#pragma unroll
                    for (int r = 0; r < CH; ++r) t.p[c + r] = plain_value<EXP, SHIFT>(e[r]);
                } else {
#pragma unroll
                    for (int r = 0; r < CH; ++r) t.p[c + r] = link_prob<EXP, SHIFT>(to_float(e[r]), true, tiny);
                }
            } else {
                bool valid[CH];
#pragma unroll
                for (int r = 0; r < CH; ++r) {
                    const int d = dd + lane - (c + r);
                    valid[r] = col_ok && d >= 0 && d < translen;
                }
                if (!EXP || batch_is_plain<CH>(e, valid)) {
#pragma unroll
                    for (int r = 0; r < CH; ++r) t.p[c + r] = valid[r] ? plain_value<EXP, SHIFT>(e[r]) : (EXP ? 0.f : DAGX_NEG_INF);
                } else {
#pragma unroll
                    for (int r = 0; r < CH; ++r) t.p[c + r] = link_prob<EXP, SHIFT>(to_float(e[r]), valid[r], tiny);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
        // pass 1: row l2 of the tile (node L_b-1-64*Jb-l2), lanes <-> r
        const int row0 = Lb - 1 - Jb * kBlk;
        TL raw[2][CH];
        auto request = [&](const int c, TL (&dst)[CH]) __attribute__((always_inline)) {
#pragma unroll
            for (int q = 0; q < CH; ++q) {
                const int row = row0 - (c + q);
                const int d = dd + (c + q) - lane;
                const bool valid = row >= 0 && d >= 0 && d < translen;
                dst[q] = at(interior || valid, row * translen + d);
            }
        };
        request(0, raw[0]);
#pragma unroll
        for (int k = 0; k < NB; ++k) {
            const int c = k * CH;
            if (k + 1 < NB) request(c + CH, raw[(k + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            const TL (&e)[CH] = raw[k & 1];
            if (interior) {   // (row0 - 63 >= 0 is the third condition of `interior`)
                if (!EXP || batch_is_plain<CH>(e)) {
#pragma unroll
                    for (int q = 0; q < CH; ++q) stage[lane][c + q] = plain_value<EXP, SHIFT>(e[q]);
                } else {
#pragma unroll
                    for (int q = 0; q < CH; ++q) stage[lane][c + q] = link_prob<EXP, SHIFT>(to_float(e[q]), true, tiny);
                }
            } else {
                bool valid[CH];
#pragma unroll
                for (int q = 0; q < CH; ++q) {
                    const int row = row0 - (c + q);
                    const int d = dd + (c + q) - lane;
                    valid[q] = row >= 0 && d >= 0 && d < translen;
                }
                if (!EXP || batch_is_plain<CH>(e, valid)) {
#pragma unroll
                    for (int q = 0; q < CH; ++q) stage[lane][c + q] = valid[q] ? plain_value<EXP, SHIFT>(e[q]) : (EXP ? 0.f : DAGX_NEG_INF);
                } else {
#pragma unroll
                    for (int q = 0; q < CH; ++q) stage[lane][c + q] = link_prob<EXP, SHIFT>(to_float(e[q]), valid[q], tiny);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // pass 2: lane <-> p_out
#pragma unroll
        for (int r = 0; r < kBlk; ++r) t.p[r] = stage[r][lane];
    }
}

}  // namespace dagx

// Fused log-softmax + gather over [B,L,V] logits, forward and in-place backward (gfx950).
//
// Both kernels are single-pass HBM streams, one workgroup per logits row:
//   forward : reads the row once (online max / sum-of-exp in registers), writes S gathered
//             log-probabilities and the row's log-sum-exp.  Algorithmic bytes per row: V*s.
//   backward: reads the row once and overwrites it with the gradient
//             -exp(x - lse) * G + (sum of g at the gathered ids).        Bytes per row: 2*V*s.
// so forward+backward move 3*V*s per row; the row is never re-read from HBM.
#include <type_traits>

#include "dagx_common.h"

namespace dagx {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 16-byte vector of T, unpacked to floats.
template <typename T> struct Pack;
template <> struct Pack<float> {
    static constexpr int N = 4;
    __device__ static __forceinline__ void unpack(const u32x4 &r, float *f) {
        f[0] = __uint_as_float(r[0]); f[1] = __uint_as_float(r[1]);
        f[2] = __uint_as_float(r[2]); f[3] = __uint_as_float(r[3]);
    }
    __device__ static __forceinline__ u32x4 pack(const float *f) {
        return u32x4{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
    }
    __device__ static __forceinline__ float max_of(const u32x4 &r) {   // largest element
        return fmaxf(fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1])), fmaxf(__uint_as_float(r[2]), __uint_as_float(r[3])));
    }
};
template <> struct Pack<__half> {
    static constexpr int N = 8;
    __device__ static __forceinline__ void unpack(const u32x4 &r, float *f) {
        const uint32_t w[4] = {r[0], r[1], r[2], r[3]};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            __half2 h = *reinterpret_cast<const __half2 *>(&w[k]);
            float2 p = __half22float2(h);
            f[2 * k] = p.x; f[2 * k + 1] = p.y;
        }
    }
    __device__ static __forceinline__ u32x4 pack(const float *f) {
        uint32_t w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            __half2 h = __floats2half2_rn(f[2 * k], f[2 * k + 1]);
            w[k] = *reinterpret_cast<uint32_t *>(&h);
        }
        return u32x4{w[0], w[1], w[2], w[3]};
    }
    // Largest element, found with packed fp16 maxima.  (Written as v_pk_max_f16 instructions:
    // __builtin_elementwise_max on _Float16 vectors compiles, with this toolchain, to its first operand.)
    __device__ static __forceinline__ uint32_t pk_max(uint32_t a, uint32_t b) {
        uint32_t o;
        asm("v_pk_max_f16 %0, %1, %2" : "=v"(o) : "v"(a), "v"(b));
        return o;
    }
    __device__ static __forceinline__ float max_of(const u32x4 &r) {
        const uint32_t m = pk_max(pk_max(r[0], r[1]), pk_max(r[2], r[3]));
        const __half2 h = *reinterpret_cast<const __half2 *>(&m);
        const float2 p = __half22float2(h);
        return fmaxf(p.x, p.y);
    }
};
template <> struct Pack<bf16_t> {
    static constexpr int N = 8;
    __device__ static __forceinline__ void unpack(const u32x4 &r, float *f) {
        const uint32_t w[4] = {r[0], r[1], r[2], r[3]};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            f[2 * k] = __uint_as_float(w[k] << 16);
            f[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
        }
    }
    __device__ static __forceinline__ u32x4 pack(const float *f) {
        uint32_t w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
            w[k] = (uint32_t)from_float<bf16_t>(f[2 * k]).bits | ((uint32_t)from_float<bf16_t>(f[2 * k + 1]).bits << 16);
        return u32x4{w[0], w[1], w[2], w[3]};
    }
    __device__ static __forceinline__ float max_of(const u32x4 &r) {
        float f[8];
        unpack(r, f);
        float m = f[0];
#pragma unroll
        for (int k = 1; k < 8; ++k) m = fmaxf(m, f[k]);
        return m;
    }
};

// Running (max, sum of exp2) in base-2 units: values are y = x*log2(e).
struct MaxSum {
    float m, s;
    __device__ __forceinline__ void merge(float om, float os) {
        float nm = fmaxf(m, om);
        if (nm > DAGX_NEG_INF) {
            s = s * fast_exp2(m - nm) + os * fast_exp2(om - nm);
            m = nm;
        }
    }
};

// Row split: [0,head) scalar elements up to a 128-byte boundary (so that the 1 KB a wave loads at a time
// covers 8 cache lines, not 9), nvec aligned vectors, scalar tail.
template <typename T>
__device__ __forceinline__ void split_row(const T *row, int64_t V, int &head, int64_t &nvec, int64_t &tail0) {
    constexpr int N = Pack<T>::N;
    uintptr_t a = reinterpret_cast<uintptr_t>(row);
    int h = (int)(((128 - (a & 127)) & 127) / sizeof(T));
    head = h < V ? h : (int)V;
    nvec = (V - head) / N;
    tail0 = head + nvec * N;
}

// ARG: also the row's arg max (lowest index among equal elements, as torch.argmax) and the largest
// log-probability max(x) - lse.  Every thread keeps its largest raw element and where it first saw it
// (an exact element index for the scalar edges, the chunk for the vector stream); once the row's
// maximum is known the threads that hold it re-read that one chunk for the exact index.
template <typename T, int BLOCK, int UNROLL, bool ARG = false>
__global__ __launch_bounds__(BLOCK) void lsg_fwd_kernel(
    const T *__restrict__ x, int L, int64_t V, int S,
    const int64_t *__restrict__ idx, int64_t is0, int64_t is1, int64_t is2,
    float *__restrict__ sel, int64_t ss0, int64_t ss1, int64_t ss2,
    float *__restrict__ lse_out, int64_t *__restrict__ argmax_out = nullptr, float *__restrict__ maxlogp_out = nullptr) {
    constexpr int N = Pack<T>::N;
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const T *xr = x + row * V;
    int head; int64_t nvec, tail0;
    split_row(xr, V, head, nvec, tail0);

    // The gathered logits are read first, with ordinary (cache-allocating) loads: when the stream
    // below reaches their cache lines it finds them in L2 instead of fetching them a second time
    // (gathering after the non-temporal stream re-reads one line per id from HBM).  Up to kPre ids
    // per thread are handled this way, the rest after the stream.
    constexpr int kPre = 2;
    const int64_t b = row / L, l = row % L;
    float pre[kPre];
#pragma unroll
    for (int u = 0; u < kPre; ++u) {
        const int s = tid + u * BLOCK;
        pre[u] = __builtin_nanf("");
        if (s < S) {
            const int64_t id = idx[b * is0 + l * is1 + (int64_t)s * is2];
            if (id >= 0 && id < V) pre[u] = to_float(xr[id]);
        }
    }

    MaxSum acc{DAGX_NEG_INF, 0.f};
    // largest raw element of this thread, the index of (or a lower bound on) its first occurrence, and
    // whether that is a chunk of the vector stream (then top_base is the chunk's first vector)
    float top = DAGX_NEG_INF;
    int top_key = 0x7fffffff;
    int64_t top_base = 0;
    bool top_vec = false;
    auto see_scalar = [&](int64_t k) __attribute__((always_inline)) {
        const float v = to_float(xr[k]);
        acc.merge(v * kLog2e, 1.f);
        if (ARG && (v > top || (v == top && (int)k < top_key))) { top = v; top_key = (int)k; top_vec = false; }
    };
    // scalar edges
    for (int64_t k = tid; k < head; k += BLOCK) see_scalar(k);
    for (int64_t k = tail0 + tid; k < V; k += BLOCK) see_scalar(k);

    const u32x4 *xv = reinterpret_cast<const u32x4 *>(xr + head);
    // Per chunk of UNROLL vectors: the largest raw element first (packed fp16 maxima for half inputs),
    // then one fused multiply-add (it converts the element and applies log2(e) and the running
    // maximum in one instruction), one exp2 and one add per element.  FULL: every slot is in range.
    auto chunk = [&](const int64_t base, auto full) __attribute__((always_inline)) {
        constexpr bool FULL = decltype(full)::value;
        u32x4 raw[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t k = base + (int64_t)u * BLOCK;
            // out-of-range slots re-read the thread's first vector and are skipped below
            raw[u] = __builtin_nontemporal_load(xv + ((FULL || k < nvec) ? k : base));
        }
        float lm = DAGX_NEG_INF;
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            if (FULL || base + (int64_t)u * BLOCK < nvec) lm = fmaxf(lm, Pack<T>::max_of(raw[u]));
        if constexpr (ARG) {
            const int key = head + (int)base * N;   // first element of the chunk: below every element of a later chunk and of the tail
            if (lm > top || (lm == top && key < top_key)) { top = lm; top_key = key; top_base = base; top_vec = true; }
        }
        const float nm = fmaxf(acc.m, lm * kLog2e);
        if (nm > DAGX_NEG_INF) {
            float part = 0.f;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                float f[N];
                Pack<T>::unpack(raw[u], f);
                float pu = 0.f;
#pragma unroll
                for (int e = 0; e < N; ++e) pu += fast_exp2(__builtin_fmaf(f[e], kLog2e, -nm));
                part += (FULL || base + (int64_t)u * BLOCK < nvec) ? pu : 0.f;
            }
            acc.s = acc.s * fast_exp2(acc.m - nm) + part;
            acc.m = nm;
        }
    };
    {
        int64_t base = tid;
        for (; base + (int64_t)(UNROLL - 1) * BLOCK < nvec; base += (int64_t)BLOCK * UNROLL) chunk(base, std::true_type{});
        if (base < nvec) chunk(base, std::false_type{});
    }

    // workgroup reduction of (m, s)
    __shared__ float sm[BLOCK / kWave], ss[BLOCK / kWave];
    __shared__ float s_lse;
    float wm = wave_max(acc.m);
    float ws = wave_sum(wm > DAGX_NEG_INF ? acc.s * fast_exp2(acc.m - wm) : 0.f);
    if ((tid & (kWave - 1)) == 0) { sm[tid / kWave] = wm; ss[tid / kWave] = ws; }
    __syncthreads();
    if (tid == 0) {
        float gm = DAGX_NEG_INF;
#pragma unroll
        for (int w = 0; w < BLOCK / kWave; ++w) gm = fmaxf(gm, sm[w]);
        float gs = 0.f;
#pragma unroll
        for (int w = 0; w < BLOCK / kWave; ++w)
            if (sm[w] > DAGX_NEG_INF) gs += ss[w] * fast_exp2(sm[w] - gm);
        // back to natural log; an all -inf row gives -inf
        float z = gm > DAGX_NEG_INF ? (gm + fast_log2(gs)) * kLn2 : DAGX_NEG_INF;
        s_lse = z;
        if (lse_out) lse_out[row] = z;
    }
    __syncthreads();
    const float z = s_lse;
    if constexpr (ARG) {
        __shared__ float top_w[BLOCK / kWave];
        __shared__ int arg_w[BLOCK / kWave];
        const float wt = wave_max(top);
        if ((tid & (kWave - 1)) == 0) top_w[tid / kWave] = wt;
        __syncthreads();
        float row_top = DAGX_NEG_INF;
#pragma unroll
        for (int w = 0; w < BLOCK / kWave; ++w) row_top = fmaxf(row_top, top_w[w]);
        int cand = 0x7fffffff;
        if (top == row_top) {
            if (!top_vec) {
                cand = top_key;
            } else {
                for (int u = UNROLL - 1; u >= 0; --u) {   // descending, so that the lowest index is assigned last
                    const int64_t k = top_base + (int64_t)u * BLOCK;
                    if (k >= nvec) continue;
                    float f[N];
                    Pack<T>::unpack(xv[k], f);
#pragma unroll
                    for (int e = N - 1; e >= 0; --e)
                        if (f[e] == row_top) cand = head + (int)k * N + e;
                }
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, kWave));
        if ((tid & (kWave - 1)) == 0) arg_w[tid / kWave] = cand;
        __syncthreads();
        if (tid == 0) {
            int first = 0x7fffffff;
#pragma unroll
            for (int w = 0; w < BLOCK / kWave; ++w) first = min(first, arg_w[w]);
            argmax_out[row] = first < V ? first : 0;
            maxlogp_out[row] = row_top - z;
        }
    }
#pragma unroll
    for (int u = 0; u < kPre; ++u) {
        const int s = tid + u * BLOCK;
        if (s < S) sel[b * ss0 + l * ss1 + (int64_t)s * ss2] = pre[u] - z;   // NaN for an id outside [0, V)
    }
    for (int s = tid + kPre * BLOCK; s < S; s += BLOCK) {
        int64_t id = idx[b * is0 + l * is1 + (int64_t)s * is2];
        float v = (id >= 0 && id < V) ? to_float(xr[id]) - z : __builtin_nanf("");
        sel[b * ss0 + l * ss1 + (int64_t)s * ss2] = v;
    }
}

// Dynamic LDS: S floats (g), S ints (ids), S floats (final value at the id), S ints (id to
// write back, -1 for later duplicates), each rounded up to a multiple of four entries.
// PATCH: the gathered positions get their scatter term inside the stream -- a bit per vocabulary entry
// says whether it is one, a small hash table (entry -> sum of its gradients) holds the terms -- so that
// the row's logits are touched by the stream alone: no separate read of each gathered logit (a cache
// line from HBM for two bytes) and no two-byte store into a line the stream has already written back
// (a read-modify-write of the line in HBM).  The same table finds the duplicates among a row's ids: every id
// is inserted once, the table keeps the lowest position that holds it and how many do; only ids
// held more than once (few, in target sequences) need the scan that sums their gradients in index
// order.  Then the dynamic LDS continues with hcap ints each of keys (-1 = empty), lowest position
// and count, hcap floats (values), S ints (positions left to scan) and V/32 + 2 words of bits; hcap
// is a power of two >= 2 S.
template <typename T, int BLOCK, int UNROLL, bool PATCH>
__global__ __launch_bounds__(BLOCK) void lsg_bwd_kernel(
    T *__restrict__ x, int L, int64_t V, int S,
    const int64_t *__restrict__ idx, int64_t is0, int64_t is1, int64_t is2,
    const float *__restrict__ gsel, int64_t gs0, int64_t gs1, int64_t gs2,
    const float *__restrict__ lse, int hcap, int hshift) {
    constexpr int N = Pack<T>::N;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int Sp = (S + 3) & ~3;   // every array starts on a 16-byte boundary
    float *g_s = reinterpret_cast<float *>(lds_raw);
    int *id_s = reinterpret_cast<int *>(g_s + Sp);
    float *fix_s = reinterpret_cast<float *>(id_s + Sp);
    int *own_s = reinterpret_cast<int *>(fix_s + Sp);
    int *hkey = own_s + Sp;
    int *hmin = hkey + hcap;
    int *hcnt = hmin + hcap;
    float *hval = reinterpret_cast<float *>(hcnt + hcap);
    int *todo = reinterpret_cast<int *>(hval + hcap);
    unsigned *bits = reinterpret_cast<unsigned *>(todo + Sp);
    __shared__ int s_ntodo;
    const unsigned hmask = (unsigned)hcap - 1u;
    auto hslot = [&](int id) -> unsigned { return ((unsigned)id * 2654435761u) >> hshift; };
    // scatter term of a gathered entry (its bit is set, so the key is in the table)
    auto patched = [&](int id) -> float {
        unsigned slot = hslot(id);
        while (hkey[slot] != id) slot = (slot + 1) & hmask;
        return hval[slot];
    };
    __shared__ float red[BLOCK / kWave];
    __shared__ float s_G;

    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    T *xr = x + row * V;
    const int64_t b = row / L, l = row % L;
    const float z2 = lse[row] * kLog2e;

    if (PATCH) {
        const int nwords = (int)(V >> 5) + 2;
        for (int k = tid; k < nwords; k += BLOCK) bits[k] = 0u;
        for (int k = tid; k < hcap; k += BLOCK) { hkey[k] = -1; hmin[k] = 0x7fffffff; hcnt[k] = 0; }
        if (tid == 0) s_ntodo = 0;
    }
    float part = 0.f;
    float x_first = 0.f;   // original logit at this thread's first gathered id: requested here, so that its
                           // round trip runs under the reduction below
    for (int s = tid; s < S; s += BLOCK) {
        float g = gsel[b * gs0 + l * gs1 + (int64_t)s * gs2];
        int64_t id = idx[b * is0 + l * is1 + (int64_t)s * is2];
        const bool ok = id >= 0 && id < V;
        if (!PATCH && s == tid && ok) x_first = to_float(xr[id]);
        g_s[s] = g;
        id_s[s] = ok ? (int)id : -1;
        part += g;
    }
    part = wave_sum(part);
    if ((tid & (kWave - 1)) == 0) red[tid / kWave] = part;
    __syncthreads();
    if (tid == 0) {
        float G = 0.f;
#pragma unroll
        for (int w = 0; w < BLOCK / kWave; ++w) G += red[w];
        s_G = G;
    }
    __syncthreads();
    const float nG = -s_G;

    if (PATCH) {
        // (the two barriers above separate the clearing of the table from its use)
        for (int s = tid; s < S; s += BLOCK) {
            const int id = id_s[s];
            if (id < 0) { own_s[s] = -1; continue; }
            unsigned slot = hslot(id);
            for (;;) {
                const int old = atomicCAS(&hkey[slot], -1, id);
                if (old == -1 || old == id) break;
                slot = (slot + 1) & hmask;
            }
            atomicMin(&hmin[slot], s);
            atomicAdd(&hcnt[slot], 1);
            own_s[s] = (int)slot;
        }
        __syncthreads();
        for (int s = tid; s < S; s += BLOCK) {
            const int slot = own_s[s];
            if (slot < 0 || hmin[slot] != s) continue;       // an id outside the row, or a later holder of an id
            const int id = id_s[s];
            if (hcnt[slot] == 1) {
                hval[slot] = g_s[s];
                atomicOr(&bits[id >> 5], 1u << (id & 31));
            } else {
                todo[atomicAdd(&s_ntodo, 1)] = s;
            }
        }
        __syncthreads();
        // ids held by several positions: one wave per id sums their gradients (every lane its positions in
        // index order, then a fixed reduction tree: the same rounding on every run)
        const int ntodo = s_ntodo;
        for (int q = tid / kWave; q < ntodo; q += BLOCK / kWave) {
            const int s = todo[q], id = id_s[s];
            float add = 0.f;
            for (int k = tid & (kWave - 1); k < S; k += kWave) add += id_s[k] == id ? g_s[k] : 0.f;
            add = wave_sum(add);
            if ((tid & (kWave - 1)) == 0) {
                hval[own_s[s]] = add;
                atomicOr(&bits[id >> 5], 1u << (id & 31));
            }
        }
        __syncthreads();
    }
    // Final value of every gathered position, from the original logit, summing duplicates in
    // index order; only the first holder of an id writes it back after the stream pass.
    // The scan reads ids and gradients four at a time (every lane the same address: LDS broadcasts).
    for (int s = tid; !PATCH && s < S; s += BLOCK) {
        const int id = id_s[s];
        const float x0 = s == tid ? x_first : (id >= 0 ? to_float(xr[id]) : 0.f);
        float add = 0.f;
        bool first = id >= 0;
        const int S4 = S & ~3;
        for (int k = 0; k < S4; k += 4) {
            const int4 ids = *reinterpret_cast<const int4 *>(id_s + k);
            const float4 gs = *reinterpret_cast<const float4 *>(g_s + k);
            const bool e0 = ids.x == id, e1 = ids.y == id, e2 = ids.z == id, e3 = ids.w == id;
            add += e0 ? gs.x : 0.f;
            add += e1 ? gs.y : 0.f;
            add += e2 ? gs.z : 0.f;
            add += e3 ? gs.w : 0.f;
            first = first && !((e0 && k < s) || (e1 && k + 1 < s) || (e2 && k + 2 < s) || (e3 && k + 3 < s));
        }
        for (int k = S4; k < S; ++k) {
            const bool same = id_s[k] == id;
            add += same ? g_s[k] : 0.f;
            first = first && !(same && k < s);
        }
        float v = 0.f;
        if (first) v = nG * fast_exp2(x0 * kLog2e - z2) + add;
        fix_s[s] = v;
        own_s[s] = first ? id : -1;
    }
    __syncthreads();

    int head; int64_t nvec, tail0;
    split_row(xr, V, head, nvec, tail0);
    auto scalar_entry = [&](int64_t k) __attribute__((always_inline)) {
        float v = nG * fast_exp2(to_float(xr[k]) * kLog2e - z2);
        if (PATCH && ((bits[k >> 5] >> (k & 31)) & 1u)) v += patched((int)k);
        xr[k] = from_float<T>(v);
    };
    for (int64_t k = tid; k < head; k += BLOCK) scalar_entry(k);
    for (int64_t k = tail0 + tid; k < V; k += BLOCK) scalar_entry(k);

    u32x4 *xv = reinterpret_cast<u32x4 *>(xr + head);
    for (int64_t base = tid; base < nvec; base += (int64_t)BLOCK * UNROLL) {
        u32x4 raw[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            int64_t k = base + (int64_t)u * BLOCK;
            raw[u] = __builtin_nontemporal_load(xv + (k < nvec ? k : base));
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            int64_t k = base + (int64_t)u * BLOCK;
            if (k < nvec) {
                float f[N];
                Pack<T>::unpack(raw[u], f);
#pragma unroll
                for (int e = 0; e < N; ++e) f[e] = nG * fast_exp2(f[e] * kLog2e - z2);
                if (PATCH) {
                    const int e0 = head + (int)k * N;            // first vocabulary entry of this vector
                    const unsigned w = (unsigned)e0 >> 5, sh = (unsigned)e0 & 31u;
                    const uint64_t two = ((uint64_t)bits[w + 1] << 32) | bits[w];
                    const unsigned hit = (unsigned)(two >> sh) & ((1u << N) - 1u);
                    if (hit) {
#pragma unroll
                        for (int e = 0; e < N; ++e)
                            if (hit & (1u << e)) f[e] += patched(e0 + e);
                    }
                }
                __builtin_nontemporal_store(Pack<T>::pack(f), xv + k);
            }
        }
    }
    if (PATCH) return;
    // All stream stores of this workgroup are complete and visible before the fix-ups land.
    __threadfence_block();
    __syncthreads();
    for (int s = tid; s < S; s += BLOCK) {
        int id = own_s[s];
        if (id >= 0) xr[id] = from_float<T>(fix_s[s]);
    }
}

// ---- host launchers -------------------------------------------------------------------------
template <typename T>
static int launch_fwd(const void *x, int B, int L, int64_t V, int S, const int64_t *idx, const int64_t *is,
                      float *sel, const int64_t *ss, float *lse, hipStream_t st, int64_t *argmax = nullptr, float *maxlogp = nullptr) {
    const int64_t rows = (int64_t)B * L;
    if (argmax) {
#define DAGX_LSG_ARG(BLK, UNR) hipLaunchKernelGGL((lsg_fwd_kernel<T, BLK, UNR, true>), dim3((unsigned)rows), dim3(BLK), 0, st, \
        static_cast<const T *>(x), L, V, S, idx, is[0], is[1], is[2], sel, ss[0], ss[1], ss[2], lse, argmax, maxlogp)
        if (V * (int64_t)sizeof(T) >= 32 * 1024) DAGX_LSG_ARG(512, 2);
        else DAGX_LSG_ARG(64, 4);
#undef DAGX_LSG_ARG
        return check_launch("lsg_fwd_argmax");
    }
    // Workgroup shape by row size (measured on MI355X at 80 KB rows: 512 threads x 2 vectors in
    // flight reads at 7.1 TB/s; 256 x 2..4 and 384 x 2 are within 2 %, 128 x 8 and 1024 x 1 lose 5-30 %).
#define DAGX_LSG_FWD(BLK, UNR) hipLaunchKernelGGL((lsg_fwd_kernel<T, BLK, UNR>), dim3((unsigned)rows), dim3(BLK), 0, st, \
        static_cast<const T *>(x), L, V, S, idx, is[0], is[1], is[2], sel, ss[0], ss[1], ss[2], lse)
    if (V * (int64_t)sizeof(T) >= 32 * 1024) DAGX_LSG_FWD(512, 2);
    else DAGX_LSG_FWD(64, 4);
#undef DAGX_LSG_FWD
    return check_launch("lsg_fwd");
}

template <typename T>
static int launch_bwd(void *x, int B, int L, int64_t V, int S, const int64_t *idx, const int64_t *is,
                      const float *g, const int64_t *gs, const float *lse, hipStream_t st) {
    const int64_t rows = (int64_t)B * L;
    size_t lds = (size_t)((S + 3) & ~3) * 16;
    // in-stream patching of the gathered entries for rows with many of them, when its bitmap and table fit beside the rest
    int hcap = 8, hshift = 29;
    while (hcap < 2 * S) { hcap *= 2; --hshift; }
    const size_t patch_lds = (size_t)hcap * 16 + (size_t)((S + 3) & ~3) * 4 + ((size_t)(V >> 5) + 2) * 4;
    // (measured at 60-80 KB rows: with 64 ids per row the scan and the late stores cost nothing and the bit test
    //  inside the stream 4-7 %; with 256 ids the scan and the late stores cost 30 %, with 512 they double the time)
    const bool patch = S >= 96 && lds + patch_lds <= 48 * 1024;
    if (patch) lds += patch_lds;
    // read+write stream: 512 threads x 4 vectors measured best at 80 KB rows (5.84 TB/s)
    // (rows with thousands of gathered ids need more dynamic LDS than a launch gets without asking)
#define DAGX_LSG_BWD(BLK, UNR, PATCH) do { \
        auto kern = lsg_bwd_kernel<T, BLK, UNR, PATCH>; \
        if (lds > 48 * 1024) { \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
            if (e != hipSuccess) { set_error("lsg_bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); return DAGX_ERR_LAUNCH; } \
        } \
        hipLaunchKernelGGL(kern, dim3((unsigned)rows), dim3(BLK), lds, st, \
        static_cast<T *>(x), L, V, S, idx, is[0], is[1], is[2], g, gs[0], gs[1], gs[2], lse, hcap, hshift); } while (0)
#define DAGX_LSG_BWD2(BLK, UNR) do { if (patch) DAGX_LSG_BWD(BLK, UNR, true); else DAGX_LSG_BWD(BLK, UNR, false); } while (0)
    if (V * (int64_t)sizeof(T) >= 32 * 1024) DAGX_LSG_BWD2(512, 4);
    else if (V * (int64_t)sizeof(T) >= 8 * 1024) DAGX_LSG_BWD2(256, 4);
    else DAGX_LSG_BWD2(64, 4);
#undef DAGX_LSG_BWD2
#undef DAGX_LSG_BWD
    return check_launch("lsg_bwd");
}

static int check_lsg_args(const void *x, int dtype, int B, int L, int64_t V, int S, const void *idx,
                          const void *is, const void *out, const void *os) {
    if (B < 0 || L < 0 || V < 1 || S < 0) { set_error("lsg: bad sizes B=%d L=%d V=%lld S=%d", B, L, (long long)V, S); return DAGX_ERR_ARGUMENT; }
    // Empty tensors own no memory: pointers are required only for what the sizes make non-empty.
    const bool rows = (int64_t)B * L > 0;
    if (rows && (!x || !is || !os || (S > 0 && (!idx || !out)))) { set_error("lsg: null pointer argument"); return DAGX_ERR_ARGUMENT; }
    if (dtype != DAGX_F32 && dtype != DAGX_F16 && dtype != DAGX_BF16) { set_error("lsg: unsupported dtype %d", dtype); return DAGX_ERR_ARGUMENT; }
    if ((int64_t)B * L > 0x7fffffffLL) { set_error("lsg: more than 2^31-1 rows"); return DAGX_ERR_UNSUPPORTED; }
    if (V > 0x7fffffffLL) { set_error("lsg: vocabulary beyond 2^31-1"); return DAGX_ERR_UNSUPPORTED; }
    if (S > 4096) { set_error("lsg: S=%d gathered ids per row exceeds the supported 4096", S); return DAGX_ERR_UNSUPPORTED; }
    return DAGX_OK;
}

}  // namespace dagx

using namespace dagx;

extern "C" int dagx_lsg_fwd(const void *logits, int dtype, int B, int L, int64_t V, int S,
                            const int64_t *idx, const int64_t idx_strides[3],
                            float *sel, const int64_t sel_strides[3], float *lse, void *stream) {
    int rc = check_lsg_args(logits, dtype, B, L, V, S, idx, idx_strides, sel, sel_strides);
    if (rc) return rc;
    if ((int64_t)B * L == 0) return DAGX_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case DAGX_F32: return launch_fwd<float>(logits, B, L, V, S, idx, idx_strides, sel, sel_strides, lse, st);
        case DAGX_F16: return launch_fwd<__half>(logits, B, L, V, S, idx, idx_strides, sel, sel_strides, lse, st);
        default: return launch_fwd<bf16_t>(logits, B, L, V, S, idx, idx_strides, sel, sel_strides, lse, st);
    }
}

extern "C" int dagx_lsg_fwd_argmax(const void *logits, int dtype, int B, int L, int64_t V, int S,
                                   const int64_t *idx, const int64_t idx_strides[3],
                                   float *sel, const int64_t sel_strides[3], float *lse,
                                   int64_t *argmax, float *max_logp, void *stream) {
    static const int64_t none[3] = {0, 0, 0};
    if (S == 0) { if (!idx_strides) idx_strides = none; if (!sel_strides) sel_strides = none; }
    int rc = check_lsg_args(logits, dtype, B, L, V, S, idx, idx_strides, sel, sel_strides);
    if (rc) return rc;
    if ((int64_t)B * L == 0) return DAGX_OK;
    if (!argmax || !max_logp) { set_error("lsg_fwd_argmax: an output pointer is null"); return DAGX_ERR_ARGUMENT; }
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case DAGX_F32: return launch_fwd<float>(logits, B, L, V, S, idx, idx_strides, sel, sel_strides, lse, st, argmax, max_logp);
        case DAGX_F16: return launch_fwd<__half>(logits, B, L, V, S, idx, idx_strides, sel, sel_strides, lse, st, argmax, max_logp);
        default: return launch_fwd<bf16_t>(logits, B, L, V, S, idx, idx_strides, sel, sel_strides, lse, st, argmax, max_logp);
    }
}

extern "C" int dagx_lsg_bwd(void *logits_inout, int dtype, int B, int L, int64_t V, int S,
                            const int64_t *idx, const int64_t idx_strides[3],
                            const float *grad_sel, const int64_t gsel_strides[3],
                            const float *lse, void *stream) {
    int rc = check_lsg_args(logits_inout, dtype, B, L, V, S, idx, idx_strides, grad_sel, gsel_strides);
    if (rc) return rc;
    if ((int64_t)B * L == 0) return DAGX_OK;
    if (!lse) { set_error("lsg_bwd: lse is null"); return DAGX_ERR_ARGUMENT; }
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case DAGX_F32: return launch_bwd<float>(logits_inout, B, L, V, S, idx, idx_strides, grad_sel, gsel_strides, lse, st);
        case DAGX_F16: return launch_bwd<__half>(logits_inout, B, L, V, S, idx, idx_strides, grad_sel, gsel_strides, lse, st);
        default: return launch_bwd<bf16_t>(logits_inout, B, L, V, S, idx, idx_strides, grad_sel, gsel_strides, lse, st);
    }
}

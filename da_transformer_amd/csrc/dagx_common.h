// Shared device/host helpers for the gfx950 DAG operator kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdlib.h>

#include "dagx.h"

namespace dagx {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
#define DAGX_NEG_INF (-__builtin_huge_valf())

// ---- element types --------------------------------------------------------------------------
struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(__half v) { return __half2float(v); }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_float<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
    uint32_t u = __float_as_uint(v);
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) { r.bits = (uint16_t)((u >> 16) | 0x40); return r; }  // NaN
    u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
    r.bits = (uint16_t)(u >> 16);
    return r;
}

// ---- fast transcendentals (v_exp_f32 / v_log_f32 work in base 2) ----------------------------
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// ---- wave-level reductions (64 lanes) ------------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

// ---- host side -----------------------------------------------------------------------------
void set_error(const char *fmt, ...);
int check_launch(const char *what);
bool force_log_domain();
bool float64_first();       // dagx_loss_fwd starts with the float64 tile sweeps (dagx_loss_float64_first)
bool redo_every_sample();   // test switch: dagx_best_alignment marks every sample as given up by the tile pipeline
size_t loss_fwd_workspace_bytes(int B, int T, int L, int translen);
size_t loss_bwd_workspace_bytes(int B);
size_t align_workspace_bytes(int B, int T, int L, int translen);
size_t align_f64_workspace_bytes(int B, int T, int L);   // the float64 alignment's score table

}  // namespace dagx

// Helpers shared by the sequence-mixer kernels of the hybrid decoders
// (norm_dyt.hip, attn_latent.hip, lightning.hip, moe.hip, seq_rows.hip,
// attn_sigmoid.hip, norm_scalar.hip, norm_rms1p.hip, attn_window.hip, mamba2.hip).
//
// Activations are bfloat16 or float32, chosen at run time by a dtype code
// (0: bf16, 1: f32); every kernel is a template over the storage type and does
// its arithmetic in f32. Small vectors (norm weights, sinks, decays, router
// corrections) are always f32.
#pragma once
#include "common.h"
#include <math.h>

template <typename T> struct Act;
template <> struct Act<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf2f(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f2bf(v); }
};
template <> struct Act<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};

// tanh through one exponential: 1 - 2 / (1 + e^{2z}); absolute error of a few
// 1e-8 over the whole range (saturates to +-1 for large |z| without overflow
// trouble: e^{2z} = inf gives 1, 0 gives -1).
__device__ __forceinline__ float tanh_f(float z) { return 1.f - 2.f / (1.f + expf(2.f * z)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
// The same through the hardware's exp2 and reciprocal (about 1 ulp each, a few
// 1e-6 relative for |z| up to 50): for results that are rounded to bfloat16.
__device__ __forceinline__ float sigmoid_fast(float z) {
  return __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.44269504088896f * z));
}
template <typename T> __device__ __forceinline__ float sigmoid_for(float z) {
  return sizeof(T) == 2 ? sigmoid_fast(z) : sigmoid_f(z);
}

static inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

// RMS norm with a weight stored around zero, and its fusion with the
// layer-scaled residual step of a pre-norm layer:
//
//   rms1p_norm_kernel:        y = x / sqrt(mean(x^2) + eps) * (1 + w)
//   scaled_add_rms1p_kernel:  resid += ls * y (per coordinate, f32, in place),
//                             h = resid / sqrt(mean(resid^2) + eps) * (1 + nxt)
//
// One workgroup per row. A row of up to 4096 entries (a multiple of 4) stays
// in registers between the statistics and the output (one read of the row);
// other widths read the row a second time. Statistics are f32; the output is
// the activation dtype or f32.
#include "seqmix.h"

#define R1_THREADS 256
#define R1_NV 4                      // float4 chunks per thread held in registers

template <typename T> struct Ld4;
template <> struct Ld4<float> {
  static __device__ __forceinline__ float4 ld(const float* p) { return *reinterpret_cast<const float4*>(p); }
  static __device__ __forceinline__ void st(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct Ld4<bf16_t> {
  static __device__ __forceinline__ float4 ld(const bf16_t* p) {
    const uint2 r = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u),
                       __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u));
  }
  static __device__ __forceinline__ void st(bf16_t* p, float4 v) {
    uint2 r;
    r.x = pack_bf16x2(v.x, v.y);
    r.y = pack_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = r;
  }
};

// TY: dtype of the sublayer output y (ignored without y); TO: dtype of h.
template <typename TY, typename TO>
__global__ __launch_bounds__(R1_THREADS) void scaled_add_rms1p_kernel(
    float* __restrict__ resid, const long* __restrict__ row_idx, const TY* __restrict__ y,
    const float* __restrict__ ls, const float* __restrict__ nxt, float eps, TO* __restrict__ h,
    int d) {
  __shared__ float scratch[R1_THREADS / 64];
  const size_t r = blockIdx.x;
  const size_t src = row_idx ? (size_t)row_idx[r] : r;
  float* xr = resid + src * d;
  const TY* yr = y ? y + src * d : nullptr;
  TO* hr = h ? h + r * d : nullptr;
  float ss = 0.f;
  if (d % 4 == 0 && d <= 4 * R1_THREADS * R1_NV) {
    float4 v[R1_NV];
#pragma unroll
    for (int i = 0; i < R1_NV; ++i) {
      const int c = 4 * (threadIdx.x + R1_THREADS * i);
      if (c < d) {
        v[i] = Ld4<float>::ld(xr + c);
        if (yr) {
          const float4 a = Ld4<TY>::ld(yr + c), s = Ld4<float>::ld(ls + c);
          v[i].x += s.x * a.x; v[i].y += s.y * a.y; v[i].z += s.z * a.z; v[i].w += s.w * a.w;
          Ld4<float>::st(xr + c, v[i]);
        }
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
      }
    }
    if (!hr) return;
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)d + eps);
#pragma unroll
    for (int i = 0; i < R1_NV; ++i) {
      const int c = 4 * (threadIdx.x + R1_THREADS * i);
      if (c < d) {
        const float4 w = Ld4<float>::ld(nxt + c);
        Ld4<TO>::st(hr + c, make_float4(v[i].x * inv * (1.f + w.x), v[i].y * inv * (1.f + w.y),
                                        v[i].z * inv * (1.f + w.z), v[i].w * inv * (1.f + w.w)));
      }
    }
    return;
  }
  for (int c = threadIdx.x; c < d; c += R1_THREADS) {
    float v = xr[c];
    if (yr) {
      v += ls[c] * Act<TY>::ld(yr + c);
      xr[c] = v;
    }
    ss += v * v;
  }
  if (!hr) return;
  ss = block_sum(ss, scratch);                 // its barriers order the writes above
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += R1_THREADS)
    Act<TO>::st(hr + c, xr[c] * inv * (1.f + nxt[c]));
}

extern "C" int loqa_rms1p_norm(const void* x, const void* row_idx, const void* w, float eps, void* y,
                               int y_dt, int rows, int d, hipStream_t st) {
  if (rows <= 0) return 0;
  if (y_dt == 0)
    hipLaunchKernelGGL((scaled_add_rms1p_kernel<float, bf16_t>), dim3(rows), dim3(R1_THREADS), 0, st,
                       (float*)x, (const long*)row_idx, (const float*)nullptr, (const float*)nullptr,
                       (const float*)w, eps, (bf16_t*)y, d);
  else
    hipLaunchKernelGGL((scaled_add_rms1p_kernel<float, float>), dim3(rows), dim3(R1_THREADS), 0, st,
                       (float*)x, (const long*)row_idx, (const float*)nullptr, (const float*)nullptr,
                       (const float*)w, eps, (float*)y, d);
  return (int)hipGetLastError();
}

extern "C" int loqa_scaled_add_rms1p(void* resid, const void* y, int y_dt, const void* ls,
                                     const void* nxt, float eps, void* h, int h_dt, int rows, int d,
                                     hipStream_t st) {
  if (rows <= 0) return 0;
  if (!nxt) h = nullptr;
#define GO(TY, TO)                                                                              \
  hipLaunchKernelGGL((scaled_add_rms1p_kernel<TY, TO>), dim3(rows), dim3(R1_THREADS), 0, st,    \
                     (float*)resid, (const long*)nullptr, (const TY*)y, (const float*)ls,       \
                     (const float*)nxt, eps, (TO*)h, d)
  if (y_dt == 0 && h_dt == 0) GO(bf16_t, bf16_t);
  else if (y_dt == 0) GO(bf16_t, float);
  else if (h_dt == 0) GO(float, bf16_t);
  else GO(float, float);
#undef GO
  return (int)hipGetLastError();
}

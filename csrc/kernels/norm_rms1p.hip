// RMS norm with a weight stored around zero, and its fusion with the
// layer-scaled residual step of a pre-norm layer:
//
//   rms1p_norm_kernel:        y = x / sqrt(mean(x^2) + eps) * (1 + w)
//   scaled_add_rms1p_kernel:  resid += ls * y (per coordinate, f32, in place),
//                             h = resid / sqrt(mean(resid^2) + eps) * (1 + nxt)
//
//   residual_rms1p_kernel:    resid += s0 y0 + s1 y1 + s2 y2 + extra (scalar scales,
//                             any of them absent), then TWO normed outputs of the
//                             same row, h_a with weight w_a and h_b with w_b: the
//                             residual step of a layer whose mixer and feed-forward
//                             run side by side on norms of the same x
//   rms_norm_cols_kernel:     y = u[:, :n] / sqrt(mean(.^2) + eps) * w, a plain-weight
//                             norm over a column slice of a fused projection
//   sigmoid_gate_kernel:      o[t, h, :Dv] *= sigmoid(gate[t, h Dv]) (heads may be padded)
//   softcap_kernel:           x <- cap tanh(x / cap)
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

// TY: dtype of the addends; TO: dtype of h_a / h_b.
template <typename TY, typename TO>
__global__ __launch_bounds__(R1_THREADS) void residual_rms1p_kernel(
    float* __restrict__ resid, const TY* __restrict__ y0, float s0, const TY* __restrict__ y1,
    float s1, const TY* __restrict__ y2, float s2, const float* __restrict__ extra,
    const float* __restrict__ wa, const float* __restrict__ wb, float eps, TO* __restrict__ ha,
    TO* __restrict__ hb, int d) {
  __shared__ float scratch[R1_THREADS / 64];
  const size_t r = blockIdx.x;
  float* xr = resid + r * d;
  const bool adds = y0 || y1 || y2 || extra;
  float ss = 0.f;
  if (d % 4 == 0 && d <= 4 * R1_THREADS * R1_NV) {
    float4 v[R1_NV];
#pragma unroll
    for (int i = 0; i < R1_NV; ++i) {
      const int c = 4 * (threadIdx.x + R1_THREADS * i);
      if (c < d) {
        v[i] = Ld4<float>::ld(xr + c);
        if (y0) { const float4 a = Ld4<TY>::ld(y0 + r * d + c);
                  v[i].x += s0 * a.x; v[i].y += s0 * a.y; v[i].z += s0 * a.z; v[i].w += s0 * a.w; }
        if (y1) { const float4 a = Ld4<TY>::ld(y1 + r * d + c);
                  v[i].x += s1 * a.x; v[i].y += s1 * a.y; v[i].z += s1 * a.z; v[i].w += s1 * a.w; }
        if (y2) { const float4 a = Ld4<TY>::ld(y2 + r * d + c);
                  v[i].x += s2 * a.x; v[i].y += s2 * a.y; v[i].z += s2 * a.z; v[i].w += s2 * a.w; }
        if (extra) { const float4 a = Ld4<float>::ld(extra + r * d + c);
                     v[i].x += a.x; v[i].y += a.y; v[i].z += a.z; v[i].w += a.w; }
        if (adds) Ld4<float>::st(xr + c, v[i]);
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
      }
    }
    if (!ha && !hb) return;
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)d + eps);
#pragma unroll
    for (int i = 0; i < R1_NV; ++i) {
      const int c = 4 * (threadIdx.x + R1_THREADS * i);
      if (c < d) {
        const float4 n = make_float4(v[i].x * inv, v[i].y * inv, v[i].z * inv, v[i].w * inv);
        if (ha) {
          const float4 w = Ld4<float>::ld(wa + c);
          Ld4<TO>::st(ha + r * d + c, make_float4(n.x * (1.f + w.x), n.y * (1.f + w.y),
                                                  n.z * (1.f + w.z), n.w * (1.f + w.w)));
        }
        if (hb) {
          const float4 w = Ld4<float>::ld(wb + c);
          Ld4<TO>::st(hb + r * d + c, make_float4(n.x * (1.f + w.x), n.y * (1.f + w.y),
                                                  n.z * (1.f + w.z), n.w * (1.f + w.w)));
        }
      }
    }
    return;
  }
  for (int c = threadIdx.x; c < d; c += R1_THREADS) {
    float v = xr[c];
    if (y0) v += s0 * Act<TY>::ld(y0 + r * d + c);
    if (y1) v += s1 * Act<TY>::ld(y1 + r * d + c);
    if (y2) v += s2 * Act<TY>::ld(y2 + r * d + c);
    if (extra) v += extra[r * d + c];
    if (adds) xr[c] = v;
    ss += v * v;
  }
  if (!ha && !hb) return;
  ss = block_sum(ss, scratch);                 // its barriers order the writes above
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += R1_THREADS) {
    const float n = xr[c] * inv;
    if (ha) Act<TO>::st(ha + r * d + c, n * (1.f + wa[c]));
    if (hb) Act<TO>::st(hb + r * d + c, n * (1.f + wb[c]));
  }
}

template <typename TU, typename TO>
__global__ __launch_bounds__(R1_THREADS) void rms_norm_cols_kernel(
    const TU* __restrict__ u, long ldu, int n, const float* __restrict__ w, float eps,
    TO* __restrict__ y) {
  __shared__ float scratch[R1_THREADS / 64];
  const size_t r = blockIdx.x;
  const TU* ur = u + r * ldu;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += R1_THREADS) {
    const float v = Act<TU>::ld(ur + c);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += R1_THREADS)
    Act<TO>::st(y + r * n + c, Act<TU>::ld(ur + c) * inv * w[c]);
}

template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(T* __restrict__ o,
                                                           const T* __restrict__ gate, long ldg,
                                                           int H, int Dvo, int Dv) {
  const size_t t = blockIdx.x;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < H * Dv; i += gridDim.y * blockDim.x) {
    const int h = i / Dv, e = i % Dv;
    T* p = o + (t * H + h) * Dvo + e;
    Act<T>::st(p, Act<T>::ld(p) * sigmoid_for<T>(Act<T>::ld(gate + t * ldg + i)));
  }
}

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, long n, float cap) {
  const float inv = 1.f / cap;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    x[i] = cap * tanhf(x[i] * inv);
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


extern "C" int loqa_residual_rms1p(void* resid, const void* y0, float s0, const void* y1, float s1,
                                   const void* y2, float s2, int y_dt, const void* extra,
                                   const void* wa, const void* wb, float eps, void* ha, void* hb,
                                   int h_dt, int rows, int d, hipStream_t st) {
  if (rows <= 0) return 0;
  if (!wa) ha = nullptr;
  if (!wb) hb = nullptr;
#define GO(TY, TO)                                                                              \
  hipLaunchKernelGGL((residual_rms1p_kernel<TY, TO>), dim3(rows), dim3(R1_THREADS), 0, st,      \
                     (float*)resid, (const TY*)y0, s0, (const TY*)y1, s1, (const TY*)y2, s2,    \
                     (const float*)extra, (const float*)wa, (const float*)wb, eps, (TO*)ha,     \
                     (TO*)hb, d)
  if (y_dt == 0 && h_dt == 0) GO(bf16_t, bf16_t);
  else if (y_dt == 0) GO(bf16_t, float);
  else if (h_dt == 0) GO(float, bf16_t);
  else GO(float, float);
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_rms_norm_cols(const void* u, int u_dt, long ldu, int n, const void* w, float eps,
                                  void* y, int y_dt, int T, hipStream_t st) {
  if (T <= 0) return 0;
  if (n <= 0 || ldu < n) return (int)hipErrorInvalidValue;
#define GO(TU, TO)                                                                             \
  hipLaunchKernelGGL((rms_norm_cols_kernel<TU, TO>), dim3(T), dim3(R1_THREADS), 0, st,         \
                     (const TU*)u, ldu, n, (const float*)w, eps, (TO*)y)
  if (u_dt == 0 && y_dt == 0) GO(bf16_t, bf16_t);
  else if (u_dt == 0) GO(bf16_t, float);
  else if (y_dt == 0) GO(float, bf16_t);
  else GO(float, float);
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_sigmoid_gate(void* o, int dt, const void* gate, long ldg, int T, int H, int Dvo,
                                 int Dv, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || Dv <= 0 || Dvo < Dv) return (int)hipErrorInvalidValue;
  const dim3 grid(T, T >= 512 ? 1 : (H * Dv + 255) / 256);
  if (dt == 0)
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, grid, dim3(256), 0, st, (bf16_t*)o,
                       (const bf16_t*)gate, ldg, H, Dvo, Dv);
  else
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, grid, dim3(256), 0, st, (float*)o,
                       (const float*)gate, ldg, H, Dvo, Dv);
  return (int)hipGetLastError();
}

extern "C" int loqa_softcap(void* x, long n, float cap, hipStream_t st) {
  if (n <= 0) return 0;
  if (!(cap > 0.f)) return (int)hipErrorInvalidValue;
  const int blocks = (int)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
  hipLaunchKernelGGL(softcap_kernel, dim3(blocks), dim3(256), 0, st, (float*)x, n, cap);
  return (int)hipGetLastError();
}

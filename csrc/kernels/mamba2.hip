// The input stage of a Mamba-2 (state-space) layer over a flat token batch.
//
// The layer's one projection is laid out z | x | B | C | dt. This launch turns
// the x | B | C columns into the inputs of the recurrence and the dt columns
// into per-token decays:
//
//   xbc[t][c] = silu(bias[c] + sum_j w[j][c] * in[t - (taps - 1 - j)][c])   (f32)
//   dt[t][h]  = softplus(u_dt[t][h] + dt_bias[h])
//   tok[t][h] = (exp(a_neg[h] * dt), dt)
//
// The convolution is causal per channel (weights tap-major, the last tap is
// the current token's). Inside a feed the earlier rows come from the batch
// itself, before the feed's first token from the sequence's tail slot
// tail[slot][taps - 1][C] (f32), and before position 0 they are zero - so a
// reused slot needs no clearing. The slot is written by seq_state_save in a
// later launch. The recurrence itself is state_scan_kernel (lightning.hip)
// with q = C, k = B, v = x, the per-token decay and the per-token value scale
// dt; everything that enters it is f32.
//
// mamba2_prep_kernel: one workgroup per token; the v8 form gives a thread 8
// neighbouring channels of a bf16 projection (16-byte loads).
#include "seqmix.h"

// The sequence of flat row t: the number of feed starts cu_q[1 .. B - 1] at or
// before t, a lane per start (all lanes must be active).
__device__ __forceinline__ int m2_seq_of_row(const int* __restrict__ cu_q, int B, int t) {
  const int lane = threadIdx.x & 63;
  int b = 0;
  for (int base = 1; base < B; base += 64) {
    const int i = base + lane;
    const bool at_or_before = i < B && cu_q[i] <= t;
    b += __popcll(__ballot(at_or_before));
  }
  return b;
}

__device__ __forceinline__ float softplus_f(float z) {
  return z > 20.f ? z : log1pf(expf(z));
}

template <typename TU>
__global__ __launch_bounds__(256) void mamba2_prep_kernel(
    const TU* __restrict__ u, long ldu, int x_off, int C, int dt_off, int Hh,
    const float* __restrict__ cw, int taps, const float* __restrict__ cb,
    const float* __restrict__ dt_bias, const float* __restrict__ a_neg,
    const float* __restrict__ tail, int nslots, const int* __restrict__ sslots,
    const int* __restrict__ cu_q, const int* __restrict__ pos, int B, float* __restrict__ xbc,
    float* __restrict__ tok) {
  const int t = blockIdx.x;
  if (t >= cu_q[B]) return;
  const int b = m2_seq_of_row(cu_q, B, t);
  const int i = t - cu_q[b], p = pos[t], keep = taps - 1;
  const float* ts = tail + (size_t)min(max(sslots[b], 0), nslots - 1) * keep * C;
  const TU* ux = u + x_off;
  if (blockIdx.y == 0)
    for (int h = threadIdx.x; h < Hh; h += blockDim.x) {
      const float dt = softplus_f(Act<TU>::ld(u + (size_t)t * ldu + dt_off + h) + dt_bias[h]);
      tok[((size_t)t * Hh + h) * 2] = expf(a_neg[h] * dt);
      tok[((size_t)t * Hh + h) * 2 + 1] = dt;
    }
  if (sizeof(TU) == 2 && C % 8 == 0 && ldu % 8 == 0 && x_off % 8 == 0) {
    for (int c = 8 * (blockIdx.y * blockDim.x + threadIdx.x); c < C; c += 8 * gridDim.y * blockDim.x) {
      float acc[8];
      {
        const float4 b0 = *reinterpret_cast<const float4*>(cb + c);
        const float4 b1 = *reinterpret_cast<const float4*>(cb + c + 4);
        acc[0] = b0.x; acc[1] = b0.y; acc[2] = b0.z; acc[3] = b0.w;
        acc[4] = b1.x; acc[5] = b1.y; acc[6] = b1.z; acc[7] = b1.w;
      }
      for (int j = 0; j < taps; ++j) {
        const int s = keep - j;                   // how many tokens back this tap reads
        if (p - s < 0) continue;                  // before the sequence's start
        float f[8];
        if (i - s >= 0) {
          unpack8(*reinterpret_cast<const uint4*>((const bf16_t*)ux + (size_t)(t - s) * ldu + c), f);
        } else {
          const float* tr = ts + (size_t)(keep + i - s) * C + c;
          const float4 a = *reinterpret_cast<const float4*>(tr);
          const float4 d = *reinterpret_cast<const float4*>(tr + 4);
          f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = d.x; f[5] = d.y; f[6] = d.z; f[7] = d.w;
        }
        const float4 w0 = *reinterpret_cast<const float4*>(cw + (size_t)j * C + c);
        const float4 w1 = *reinterpret_cast<const float4*>(cw + (size_t)j * C + c + 4);
        acc[0] += w0.x * f[0]; acc[1] += w0.y * f[1]; acc[2] += w0.z * f[2]; acc[3] += w0.w * f[3];
        acc[4] += w1.x * f[4]; acc[5] += w1.y * f[5]; acc[6] += w1.z * f[6]; acc[7] += w1.w * f[7];
      }
      float* o = xbc + (size_t)t * C + c;
      *reinterpret_cast<float4*>(o) =
          make_float4(silu_f(acc[0]), silu_f(acc[1]), silu_f(acc[2]), silu_f(acc[3]));
      *reinterpret_cast<float4*>(o + 4) =
          make_float4(silu_f(acc[4]), silu_f(acc[5]), silu_f(acc[6]), silu_f(acc[7]));
    }
    return;
  }
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float acc = cb[c];
    for (int j = 0; j < taps; ++j) {
      const int s = keep - j;
      if (p - s < 0) continue;
      const float uv = i - s >= 0 ? Act<TU>::ld(ux + (size_t)(t - s) * ldu + c)
                                  : ts[(size_t)(keep + i - s) * C + c];
      acc += cw[(size_t)j * C + c] * uv;
    }
    xbc[(size_t)t * C + c] = silu_f(acc);
  }
}

extern "C" int loqa_mamba2_prep(const void* u, int u_dt, long ldu, int x_off, int C, int dt_off,
                                int Hh, const void* cw, int taps, const void* cb,
                                const void* dt_bias, const void* a_neg, const void* tail, int nslots,
                                const void* sslots, const void* cu_q, const void* pos, int B, int T,
                                void* xbc, void* tok, hipStream_t st) {
  if (T <= 0) return 0;
  if (B <= 0 || taps < 1 || nslots <= 0 || C <= 0 || Hh <= 0) return (int)hipErrorInvalidValue;
  // few rows: spread a row's channels over several workgroups
  const int per = u_dt == 0 && C % 8 == 0 ? 8 * 256 : 256;
  const dim3 grid(T, T >= 512 ? 1 : (C + per - 1) / per);
#define GO(TU)                                                                                  \
  hipLaunchKernelGGL(mamba2_prep_kernel<TU>, grid, dim3(256), 0, st, (const TU*)u, ldu, x_off, C, \
                     dt_off, Hh, (const float*)cw, taps, (const float*)cb,                      \
                     (const float*)dt_bias, (const float*)a_neg, (const float*)tail, nslots,    \
                     (const int*)sslots, (const int*)cu_q, (const int*)pos, B, (float*)xbc,     \
                     (float*)tok)
  if (u_dt == 0) GO(bf16_t); else GO(float);
#undef GO
  return (int)hipGetLastError();
}

// A matrix memory with exponential gates and a running-maximum stabiliser
// (mLSTM) over a flat token batch. Per sequence and head, with log gates li, lf:
//
//   m_t = max(lf_t + m_{t-1}, li_t)                       (m = 0 before position 0)
//   S_t = exp(lf_t + m_{t-1} - m_t) S_{t-1} + exp(li_t - m_t) k_t v_t^T
//   n_t = the same recurrence with k_t alone
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//
// The matrix recurrence is state_scan_kernel (lightning.hip) with a per-token
// decay and a per-token input scale; the value rows carry one more column that
// is constantly 1, so the state's last column IS n and the scan's last output
// column is n . q. This file holds what surrounds the scan:
//
// exp_gate_scan_kernel: one wave per (sequence, head). 64 tokens at a time, a
// lane per token, compute the log gates (tanh cap, log-sigmoid) in parallel;
// the running maximum then walks the 64 tokens in order with wave-uniform
// reads of the lanes' gates - the same f32 operations in the same order as a
// token-by-token evaluation, whatever the cut of the prompt - and each lane
// turns its token's (m_{t-1}, m_t) into the decay, the input scale and the
// floor exp(-m_t). The last m goes to the sequence's slot.
//
// matrix_memory_inputs_kernel: q D^(-1/2) | k | per head (v, 1) in f32.
//
// normalized_gated_rmsnorm_kernel: one wave per (token, head): the division
// by the normaliser, the head's RMS norm, the weight and the sigmoid gate.
#include "seqmix.h"

__device__ __forceinline__ float log_sigmoid_f(float x) {
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

__global__ __launch_bounds__(64) void exp_gate_scan_kernel(
    const float* __restrict__ gz, int H, const float* __restrict__ ib,
    const float* __restrict__ fb, float cap, float* __restrict__ m_state, int nslots,
    const int* __restrict__ sslots, const int* __restrict__ cu_q, const int* __restrict__ pos,
    float* __restrict__ tok, float* __restrict__ floor_out) {
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (q1 <= q0) return;
  float* ms = m_state + (size_t)min(max(sslots[b], 0), nslots - 1) * H + h;
  float m = pos[q0] == 0 ? 0.f : *ms;          // wave-uniform
  const float bi = ib[h], bf = fb[h], icap = 1.f / cap;
  for (int t0 = q0; t0 < q1; t0 += 64) {
    const int t = t0 + lane;
    const bool ok = t < q1;
    float li = 0.f, lf = 0.f;
    if (ok) {
      li = cap * tanhf((gz[(size_t)t * 2 * H + h] + bi) * icap);
      lf = log_sigmoid_f(cap * tanhf((gz[(size_t)t * 2 * H + H + h] + bf) * icap));
    }
    const int nt = min(64, q1 - t0);
    float m_prev = 0.f, m_mine = 0.f;
    for (int j = 0; j < nt; ++j) {
      // j is wave-uniform: scalar lane reads, no trip through the LDS crossbar
      const float lij = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(li), j));
      const float lfj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lf), j));
      const float m1 = fmaxf(lfj + m, lij);
      if (lane == j) { m_prev = m; m_mine = m1; }
      m = m1;
    }
    if (ok) {
      tok[((size_t)t * H + h) * 2] = expf(lf + m_prev - m_mine);
      tok[((size_t)t * H + h) * 2 + 1] = expf(li - m_mine);
      floor_out[(size_t)t * H + h] = expf(-m_mine);
    }
  }
  if (lane == 0) *ms = m;
}

template <typename TU>
__global__ __launch_bounds__(256) void matrix_memory_inputs_kernel(const TU* __restrict__ u, long ldu,
                                                                   int H, int D, int Dv,
                                                                   float* __restrict__ act) {
  const size_t t = blockIdx.x;
  const int HD = H * D, n = 2 * HD + H * (Dv + 1);
  const float qs = 1.f / sqrtf((float)D);
  const TU* ur = u + t * ldu;
  float* ar = act + t * n;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < n; c += gridDim.y * blockDim.x) {
    float v;
    if (c < HD) v = Act<TU>::ld(ur + c) * qs;
    else if (c < 2 * HD) v = Act<TU>::ld(ur + c);
    else {
      const int hh = (c - 2 * HD) / (Dv + 1), e = (c - 2 * HD) % (Dv + 1);
      v = e < Dv ? Act<TU>::ld(ur + 2 * HD + hh * Dv + e) : 1.f;
    }
    ar[c] = v;
  }
}

template <typename TG, typename TO>
__global__ __launch_bounds__(64) void normalized_gated_rmsnorm_kernel(
    const float* __restrict__ o, const float* __restrict__ floor_in, const float* __restrict__ w,
    const TG* __restrict__ gate, long ldg, float eps, TO* __restrict__ y, int H, int Dv) {
  const size_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* oh = o + (t * H + h) * (Dv + 1);
  const float den = fmaxf(fabsf(oh[Dv]), floor_in[t * H + h]) + 1e-6f;
  float ss = 0.f;
  for (int e = lane; e < Dv; e += 64) {
    const float v = oh[e] / den;
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)Dv + eps);
  for (int e = lane; e < Dv; e += 64) {
    const int c = h * Dv + e;
    const float g = Act<TG>::ld(gate + t * ldg + c);
    Act<TO>::st(y + t * H * Dv + c, oh[e] / den * inv * w[c] * sigmoid_f(g));
  }
}

extern "C" int loqa_exp_gate_scan(const void* gz, int H, const void* ib, const void* fb, float cap,
                                  void* m_state, int nslots, const void* sslots, const void* cu_q,
                                  const void* pos, int B, int T, void* tok, void* floor_out,
                                  hipStream_t st) {
  if (T <= 0 || B <= 0) return 0;
  if (H <= 0 || nslots <= 0 || !(cap > 0.f)) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(exp_gate_scan_kernel, dim3(B, H), dim3(64), 0, st, (const float*)gz, H,
                     (const float*)ib, (const float*)fb, cap, (float*)m_state, nslots,
                     (const int*)sslots, (const int*)cu_q, (const int*)pos, (float*)tok,
                     (float*)floor_out);
  return (int)hipGetLastError();
}

extern "C" int loqa_matrix_memory_inputs(const void* u, int u_dt, long ldu, int H, int D, int Dv,
                                         void* act, int T, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || D <= 0 || Dv <= 0) return (int)hipErrorInvalidValue;
  const int n = 2 * H * D + H * (Dv + 1);
  const dim3 grid(T, T >= 512 ? 1 : (n + 255) / 256);
  if (u_dt == 0)
    hipLaunchKernelGGL(matrix_memory_inputs_kernel<bf16_t>, grid, dim3(256), 0, st,
                       (const bf16_t*)u, ldu, H, D, Dv, (float*)act);
  else
    hipLaunchKernelGGL(matrix_memory_inputs_kernel<float>, grid, dim3(256), 0, st, (const float*)u,
                       ldu, H, D, Dv, (float*)act);
  return (int)hipGetLastError();
}

extern "C" int loqa_normalized_gated_rmsnorm(const void* o, const void* floor_in, const void* w,
                                             const void* gate, int g_dt, long ldg, float eps,
                                             void* y, int y_dt, int T, int H, int Dv,
                                             hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || Dv <= 0) return (int)hipErrorInvalidValue;
#define GO(TG, TO)                                                                             \
  hipLaunchKernelGGL((normalized_gated_rmsnorm_kernel<TG, TO>), dim3(T, H), dim3(64), 0, st,    \
                     (const float*)o, (const float*)floor_in, (const float*)w, (const TG*)gate, \
                     ldg, eps, (TO*)y, H, Dv)
  if (g_dt == 0 && y_dt == 0) GO(bf16_t, bf16_t);
  else if (g_dt == 0) GO(bf16_t, float);
  else if (y_dt == 0) GO(float, bf16_t);
  else GO(float, float);
#undef GO
  return (int)hipGetLastError();
}

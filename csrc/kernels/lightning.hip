// Linear recurrences with a carried matrix state - decayed linear attention
// ("lightning") and the Mamba-2 state-space recurrence - and the gated RMS norm
// that follows them.
//
// Per sequence and head:  S_t = a_t * S_{t-1} + k_t (c_t v_t)^T,
//                         o_t = S_t^T q_t + skip_h v_t.
// S [D, Dv] lives in f32 state slots between steps. Lightning attention: a_t =
// decay_h, c_t = 1, no skip, q / k / v = SiLU of the projection columns, each
// head with its own q and k. Mamba-2: a_t = exp(-exp(A_log_h) dt_t) and c_t =
// dt_t per token (tok[t][h] = (a, c)), q = C_t and k = B_t shared by `hpg`
// neighbouring heads, v = x_t, skip = D_h.
//
// lightning_prep_kernel: act = SiLU of the q | k | v projection columns, f32,
// once per step (every column block of a head reads the same q and k).
//
// state_scan_kernel: one workgroup per (sequence, head, EC value columns).
// The columns of S evolve independently, so the grid splits Dv freely: EC is
// 32 when the batch alone fills the GPU and 16 or 8 for a lone prompt. A
// thread holds S[d, e] for one column e and a contiguous run of MAXD rows d in
// registers (16 threads per column). The step's tokens are staged TC at a time
// in LDS (rows zero-padded to 16 MAXD so the recurrence reads them as float4);
// the values of the next two token groups are already in flight in registers while
// the current one is processed. The recurrence runs token by token in f32 in
// the order of the definition; only the S updates chain from token to token,
// the next token's k / q / v are read from LDS while this token is computed,
// and the 16 row-partials of o_t are written to LDS and summed in a fixed
// order after each group. A prompt portion, a single decode token, or any cut
// of a prompt gives the same bits (for a given EC: the column split does not
// change any sum).
#include "seqmix.h"
#include <type_traits>

#define LS_DP 16        // row partitions (threads per column)

template <typename T>
__global__ __launch_bounds__(256) void lightning_prep_kernel(const T* __restrict__ qkv, long ld,
                                                             int n, float* __restrict__ act) {
  const size_t r = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < n; c += gridDim.y * blockDim.x)
    act[r * n + c] = silu_f(Act<T>::ld(qkv + r * ld + c));
}

template <int MAXD, int TC, int EC>   // D <= LS_DP * MAXD
__global__ __launch_bounds__(EC * LS_DP) void state_scan_kernel(
    const float* __restrict__ act, long ld, int H, int D, int Dv, int q_off, int k_off, int v_off,
    int hpg, float* __restrict__ state, const int* __restrict__ state_slots,
    const int* __restrict__ cu_q, const int* __restrict__ positions,
    const float* __restrict__ decay, const float* __restrict__ tok, const float* __restrict__ skip,
    float* __restrict__ o) {
  constexpr int NTH = EC * LS_DP;
  constexpr int DPAD = LS_DP * MAXD;            // padded row length in LDS
  constexpr int NPT = TC * DPAD / NTH;          // staged q (and k) values per thread
  constexpr int NVT = (TC * EC + NTH - 1) / NTH;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;                         // [TC][DPAD]
  float* ks = qs + TC * DPAD;              // [TC][DPAD]
  float* vs = ks + TC * DPAD;              // [TC][EC]
  float* red = vs + TC * EC;               // [TC][LS_DP][EC]
  float* lams = red + TC * LS_DP * EC;     // [TC] the tokens' decays
  float* vsc = lams + TC;                  // [TC] the tokens' value scales
  const int b = blockIdx.x, h = blockIdx.y, e0 = blockIdx.z * EC;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (q1 <= q0) return;
  const int tid = threadIdx.x;
  const int e = tid % EC, dp = tid / EC;
  const bool col = e0 + e < Dv;
  const float lamc = decay ? decay[h] : 1.f;
  const float sk = skip ? skip[h] : 0.f;
  float* Sg = state + (((size_t)state_slots[b] * H + h) * D) * Dv + e0 + e;
  const bool fresh = positions[q0] == 0;
  float S[MAXD];
#pragma unroll
  for (int i = 0; i < MAXD; ++i) {
    const int d = dp * MAXD + i;
    S[i] = (!fresh && col && d < D) ? Sg[(size_t)d * Dv] : 0.f;
  }
  const size_t qoff = (size_t)q_off + (size_t)(h / hpg) * D;
  const size_t koff = (size_t)k_off + (size_t)(h / hpg) * D;
  const size_t voff = (size_t)v_off + (size_t)h * Dv + e0;
  // Two register sets: while token group g is processed, the loads of groups
  // g + 1 and g + 2 are in flight.
  float rq[2][NPT], rk[2][NPT], rv[2][NVT], rl[2], rc[2];
  auto fetch = [&](auto BUF, int t0) {     // activations of tokens t0 .. t0 + TC
    constexpr int U = decltype(BUF)::value;
    if (tid < TC) {
      const bool ok = tok && t0 + tid < q1;
      rl[U] = ok ? tok[((size_t)(t0 + tid) * H + h) * 2] : lamc;
      rc[U] = ok ? tok[((size_t)(t0 + tid) * H + h) * 2 + 1] : 1.f;
    }
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
      const int i = tid + NTH * j, tt = i / DPAD, d = i % DPAD;
      const bool ok = t0 + tt < q1 && d < D;
      const float* row = act + (size_t)(ok ? t0 + tt : q0) * ld;
      rq[U][j] = ok ? row[qoff + d] : 0.f;
      rk[U][j] = ok ? row[koff + d] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NVT; ++j) {
      const int i = tid + NTH * j, tt = i / EC, c = i % EC;
      const bool ok = i < TC * EC && t0 + tt < q1 && e0 + c < Dv;
      rv[U][j] = ok ? act[(size_t)(t0 + tt) * ld + voff + c] : 0.f;
    }
  };
  auto group = [&](auto BUF, int t0) {
    constexpr int U = decltype(BUF)::value;
    const int nt = min(TC, q1 - t0);
    __syncthreads();                       // the previous group's LDS is consumed
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
      qs[tid + NTH * j] = rq[U][j];
      ks[tid + NTH * j] = rk[U][j];
    }
#pragma unroll
    for (int j = 0; j < NVT; ++j)
      if (tid + NTH * j < TC * EC) vs[tid + NTH * j] = rv[U][j];
    if (tid < TC) { lams[tid] = rl[U]; vsc[tid] = rc[U]; }
    __syncthreads();
    if (t0 + 2 * TC < q1) fetch(BUF, t0 + 2 * TC);   // this set is free again
    float4 kc[MAXD / 4], qc[MAXD / 4];
    float vc;
    {
      const float4* k4 = reinterpret_cast<const float4*>(ks + dp * MAXD);
      const float4* q4 = reinterpret_cast<const float4*>(qs + dp * MAXD);
#pragma unroll
      for (int i = 0; i < MAXD / 4; ++i) { kc[i] = k4[i]; qc[i] = q4[i]; }
      vc = vs[e];
    }
    for (int tt = 0; tt < nt; ++tt) {
      float4 kn[MAXD / 4], qn[MAXD / 4];
      float vn = 0.f;
      const int tn = tt + 1 < nt ? tt + 1 : tt;          // clamped: the last read is a repeat
      {
        const float4* k4 = reinterpret_cast<const float4*>(ks + tn * DPAD + dp * MAXD);
        const float4* q4 = reinterpret_cast<const float4*>(qs + tn * DPAD + dp * MAXD);
#pragma unroll
        for (int i = 0; i < MAXD / 4; ++i) { kn[i] = k4[i]; qn[i] = q4[i]; }
        vn = vs[tn * EC + e];
      }
      float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
      const float lam = lams[tt], vw = vc * vsc[tt];
#pragma unroll
      for (int i = 0; i < MAXD / 4; ++i) {
        S[4 * i] = lam * S[4 * i] + kc[i].x * vw;         p0 += S[4 * i] * qc[i].x;
        S[4 * i + 1] = lam * S[4 * i + 1] + kc[i].y * vw; p1 += S[4 * i + 1] * qc[i].y;
        S[4 * i + 2] = lam * S[4 * i + 2] + kc[i].z * vw; p2 += S[4 * i + 2] * qc[i].z;
        S[4 * i + 3] = lam * S[4 * i + 3] + kc[i].w * vw; p3 += S[4 * i + 3] * qc[i].w;
      }
      red[(tt * LS_DP + dp) * EC + e] = (p0 + p1) + (p2 + p3);
#pragma unroll
      for (int i = 0; i < MAXD / 4; ++i) { kc[i] = kn[i]; qc[i] = qn[i]; }
      vc = vn;
    }
    __syncthreads();
    for (int i = tid; i < nt * EC; i += NTH) {
      const int tt = i / EC, c = i % EC;
      if (e0 + c < Dv) {
        const float* r = red + tt * LS_DP * EC + c;
        float sum = r[0];
#pragma unroll
        for (int w = 1; w < LS_DP; ++w) sum += r[w * EC];
        if (skip) sum += sk * vs[tt * EC + c];
        o[(size_t)(t0 + tt) * H * Dv + (size_t)h * Dv + e0 + c] = sum;
      }
    }
  };
  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  fetch(B0{}, q0);
  if (q0 + TC < q1) fetch(B1{}, q0 + TC);
  for (int t0 = q0; t0 < q1; t0 += 2 * TC) {
    group(B0{}, t0);
    if (t0 + TC < q1) group(B1{}, t0 + TC);
  }
#pragma unroll
  for (int i = 0; i < MAXD; ++i) {
    const int d = dp * MAXD + i;
    if (col && d < D) Sg[(size_t)d * Dv] = S[i];
  }
}

// y = rmsnorm(o) * w * sigmoid(gate) (mode 0), rmsnorm(o * silu(gate)) * w (mode
// 1: the gate before the norm) or rmsnorm(o) * w * silu(gate) (mode 2); a row is
// normalised in `groups` equal parts, each by its own root mean square. One
// workgroup per (row, part).
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(
    const float* __restrict__ o, const float* __restrict__ w, const TG* __restrict__ gate, long ldg,
    float eps, TO* __restrict__ y, int n, int groups, int mode) {
  __shared__ float scratch[4];
  const size_t r = blockIdx.x;
  const int per = n / groups, c0 = blockIdx.y * per;
  const bool silu_first = mode == 1;
  float ss = 0.f;
  for (int c = c0 + threadIdx.x; c < c0 + per; c += blockDim.x) {
    float v = o[r * n + c];
    if (silu_first) v *= silu_f(Act<TG>::ld(gate + r * ldg + c));
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)per + eps);
  for (int c = c0 + threadIdx.x; c < c0 + per; c += blockDim.x) {
    const float g = Act<TG>::ld(gate + r * ldg + c);
    const float v = o[r * n + c];
    Act<TO>::st(y + r * n + c, silu_first ? v * silu_f(g) * inv * w[c]
                                          : v * inv * w[c] * (mode == 2 ? silu_f(g) : sigmoid_f(g)));
  }
}

extern "C" int loqa_lightning_prep(const void* qkv, int dt, long ld, int T, int n, void* act,
                                   hipStream_t st) {
  if (T <= 0 || n <= 0) return 0;
  const dim3 grid(T, T >= 512 ? 1 : (n + 255) / 256);
  if (dt == 0)
    hipLaunchKernelGGL(lightning_prep_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)qkv, ld, n,
                       (float*)act);
  else
    hipLaunchKernelGGL(lightning_prep_kernel<float>, grid, dim3(256), 0, st, (const float*)qkv, ld, n,
                       (float*)act);
  return (int)hipGetLastError();
}

// act: f32 [T, ld]; head h reads q at q_off + (h / hpg) D, k at k_off + (h / hpg) D,
// v at v_off + h Dv. Exactly one of decay [H] and tok [T, H, 2] is given.
extern "C" int loqa_state_scan(const void* act, long ld, int H, int D, int Dv, int q_off, int k_off,
                               int v_off, int hpg, void* state, int nslots,
                               const void* state_slots, const void* cu_q, const void* positions,
                               const void* decay, const void* tok, const void* skip, void* o, int B,
                               int T, int col_block, hipStream_t st) {
  if (T <= 0 || B <= 0) return 0;
  if (D > LS_DP * 16 || D <= 0 || Dv <= 0 || hpg <= 0 || H % hpg || (!decay) == (!tok))
    return (int)hipErrorInvalidValue;
  (void)nslots;
  // column block: 32 when (sequences x heads x column blocks) fill the GPU,
  // narrower for a lone prompt
  const long wg32 = (long)B * H * ((Dv + 31) / 32);
  int ec = wg32 >= 192 ? 32 : (wg32 * 2 >= 192 ? 16 : 8);
  // a caller that runs other work beside the scan may ask for denser workgroups
  if (col_block == 8 || col_block == 16 || col_block == 32) ec = col_block;
#define GO(MD, TCC, ECC)                                                                          \
  hipLaunchKernelGGL((state_scan_kernel<MD, TCC, ECC>), dim3(B, H, (Dv + ECC - 1) / ECC),         \
                     dim3(ECC * LS_DP),                                                           \
                     (size_t)(2 * TCC * LS_DP * MD + TCC * ECC + TCC * LS_DP * ECC + 2 * TCC) * 4, \
                     st, (const float*)act, ld, H, D, Dv, q_off, k_off, v_off, hpg, (float*)state, \
                     (const int*)state_slots, (const int*)cu_q, (const int*)positions,            \
                     (const float*)decay, (const float*)tok, (const float*)skip, (float*)o)
#define GOE(MD, TCC)                                                                              \
  do {                                                                                            \
    if (ec == 32) GO(MD, TCC, 32); else if (ec == 16) GO(MD, TCC, 16); else GO(MD, TCC, 8);       \
  } while (0)
  if (D <= 64) GOE(4, 16);
  else if (D <= 128) GOE(8, 16);
  else GOE(16, 8);
#undef GOE
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_gated_rmsnorm(const void* o, const void* w, const void* gate, int g_dt, long ldg,
                                  float eps, void* y, int y_dt, int T, int n, int groups,
                                  int mode, hipStream_t st) {
  if (T <= 0) return 0;
  if (groups <= 0 || n % groups) return (int)hipErrorInvalidValue;
#define GO(TG, TO)                                                                            \
  hipLaunchKernelGGL((gated_rmsnorm_kernel<TG, TO>), dim3(T, groups), dim3(256), 0, st,        \
                     (const float*)o, (const float*)w, (const TG*)gate, ldg, eps, (TO*)y, n,   \
                     groups, mode)
  if (g_dt == 0 && y_dt == 0) GO(bf16_t, bf16_t);
  else if (g_dt == 0) GO(bf16_t, float);
  else if (y_dt == 0) GO(float, bf16_t);
  else GO(float, float);
#undef GO
  return (int)hipGetLastError();
}

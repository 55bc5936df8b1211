// The gated delta rule over a flat token batch. Per sequence and head, with a
// decay g_t and a write strength beta_t per token:
//
//   S <- g_t S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
//
// delta_prep_kernel: the input stage, a wave per (token, run of D channels). The
// q | k | v columns of the projected row pass a causal convolution per channel
// (weights tap-major, the last tap is the current token's, no bias; rows before
// the feed from the sequence's tail slot, zeros before position 0, so a reused
// slot needs no clearing) and SiLU; a run that is a q or k head is made a unit
// vector x / sqrt(sum x^2 + 1e-6) by one wave reduction (q also times D^(-1/2)).
// The gate rows give beta = sigmoid(z) and g = exp(a_neg softplus(z + dt_bias)).
// Everything it writes is f32.
//
// delta_scan_kernel: one workgroup per (sequence, head, EC value columns). A
// column of S never meets another column: u_e depends on column e of S only.
// Sixteen neighbouring lanes (thirty-two when there are more than 64 rows)
// share a column, each holding a contiguous run of MAXD of its D rows in
// registers, so that the two products with the OLD state that a token needs,
// S^T k and S^T q, are MAXD multiply-adds per lane and one lane-group sum each
// through data-parallel moves and, across the two 16-lane rows, the swizzle
// network (no LDS memory, no barrier):
//
//   r = S^T k,  s = S^T q,  c = k . q        (before this token's update)
//   u = beta (v - g r),   o = g s + u c,   S <- g S + k u
//
// which is the definition with the read-out folded in (S_new^T q = g S^T q + u
// k . q). c is the same for every column: it is computed once per token group.
// The decayed state g S is formed while the sum for r is under way, so that one
// multiply-add per row follows it. The state is stored with a column's rows side by side ([slots, H, Dv,
// D]), so a wave reads and writes 4 D contiguous floats. The step's tokens are
// staged TC at a time in LDS (rows zero-padded to 16 MAXD), the next group's
// values already in flight in registers. The recurrence runs token by token
// in f32; a prompt portion, a single token or any cut of a prompt is the same
// sequence of operations, for any EC.
#include "seqmix.h"
#include <type_traits>

#define DR_DP 16        // lanes per state column

__device__ __forceinline__ int dr_seq_of_row(const int* __restrict__ cu_q, int B, int t) {
  const int lane = threadIdx.x & 63;
  int b = 0;
  for (int base = 1; base < B; base += 64) {
    const int i = base + lane;
    const bool at_or_before = i < B && cu_q[i] <= t;
    b += __popcll(__ballot(at_or_before));
  }
  return b;
}

__device__ __forceinline__ float dr_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <int CTRL> __device__ __forceinline__ float dr_dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
// the sum over each run of 16 lanes, in every lane of the run
__device__ __forceinline__ float dr_sum16(float v) {
  v += dr_dpp<0xB1>(v);              // lanes 1 0 3 2 of each four
  v += dr_dpp<0x4E>(v);              // lanes 2 3 0 1 of each four
  v += dr_dpp<0x141>(v);             // the other four of each eight (mirror)
  v += dr_dpp<0x140>(v);             // the other eight of each sixteen (mirror)
  return v;
}

// the sum over each run of LPC = 16 or 32 lanes, in every lane of the run; the
// step across the two 16-lane rows goes through the swizzle network
template <int LPC> __device__ __forceinline__ float dr_lane_sum(float v) {
  v = dr_sum16(v);
  if (LPC == 32)
    v += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));   // lane ^ 16
  return v;
}

template <typename TU>
__global__ __launch_bounds__(64) void delta_prep_kernel(
    const TU* __restrict__ u, long ldu, const float* __restrict__ gz, int G, int D, int H, int Dv,
    const float* __restrict__ cw, int taps, const float* __restrict__ tail, int nslots,
    const float* __restrict__ a_neg, const float* __restrict__ dt_bias,
    const int* __restrict__ sslots, const int* __restrict__ cu_q, const int* __restrict__ pos,
    int B, float* __restrict__ act, float* __restrict__ tok) {
  const int t = blockIdx.x, lane = threadIdx.x;
  if (t >= cu_q[B]) return;
  const int b = dr_seq_of_row(cu_q, B, t);
  const int i = t - cu_q[b], p = pos[t], keep = taps - 1;
  const int QK = 2 * G * D, C = QK + H * Dv;
  const float* ts = tail + (size_t)min(max(sslots[b], 0), nslots - 1) * keep * C;
  if (blockIdx.y == 0)
    for (int h = lane; h < H; h += 64) {
      const float* z = gz + (size_t)t * 2 * H;
      tok[((size_t)t * H + h) * 2] = expf(a_neg[h] * dr_softplus(z[H + h] + dt_bias[h]));
      tok[((size_t)t * H + h) * 2 + 1] = sigmoid_f(z[h]);
    }
  const float qscale = 1.f / sqrtf((float)D);
  const int units = (C + D - 1) / D;            // runs of D channels: the q heads, the k heads, then v
  constexpr int NC = 8;                         // channels per lane (D <= 512)
  for (int un = blockIdx.y; un < units; un += gridDim.y) {
    const int c0 = un * D, n = min(D, C - c0);
    float y[NC];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      const int c = c0 + lane + 64 * k;
      y[k] = 0.f;
      if (lane + 64 * k < n) {
        float acc = 0.f;
        for (int j = 0; j < taps; ++j) {
          const int s = keep - j;               // how many tokens back this tap reads
          if (p - s < 0) continue;              // before the sequence's start
          const float uv = i - s >= 0 ? Act<TU>::ld(u + (size_t)(t - s) * ldu + c)
                                      : ts[(size_t)(keep + i - s) * C + c];
          acc += cw[(size_t)j * C + c] * uv;
        }
        y[k] = silu_f(acc);
        ss += y[k] * y[k];
      }
    }
    float mul = 1.f;
    if (c0 < QK) {                              // a q or k head: unit length (q also D^(-1/2))
      ss = wave_sum(ss);
      mul = (c0 < G * D ? qscale : 1.f) / sqrtf(ss + 1e-6f);
    }
#pragma unroll
    for (int k = 0; k < NC; ++k)
      if (lane + 64 * k < n) act[(size_t)t * C + c0 + lane + 64 * k] = y[k] * mul;
  }
}

// The same stage for bfloat16 rows whose heads are a power-of-two number (up
// to 64) of 16-byte runs: a lane owns 8 neighbouring channels (one 16-byte
// load per tap, 32-byte stores), the D / 8 lanes of a head add up their
// squares through data-parallel moves, a wave covers 512 channels.
__device__ __forceinline__ float dr_group_sum(float v, int gs) {
  if (gs >= 2) v += dr_dpp<0xB1>(v);
  if (gs >= 4) v += dr_dpp<0x4E>(v);
  if (gs >= 8) v += dr_dpp<0x141>(v);
  if (gs >= 16) v += dr_dpp<0x140>(v);
  if (gs >= 32) v += __shfl_xor(v, 16, 64);
  if (gs >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

__global__ __launch_bounds__(64) void delta_prep_v8_kernel(
    const bf16_t* __restrict__ u, long ldu, const float* __restrict__ gz, int G, int D, int H, int Dv,
    const float* __restrict__ cw, int taps, const float* __restrict__ tail, int nslots,
    const float* __restrict__ a_neg, const float* __restrict__ dt_bias,
    const int* __restrict__ sslots, const int* __restrict__ cu_q, const int* __restrict__ pos,
    int B, float* __restrict__ act, float* __restrict__ tok) {
  const int t = blockIdx.x, lane = threadIdx.x;
  if (t >= cu_q[B]) return;
  const int b = dr_seq_of_row(cu_q, B, t);
  const int i = t - cu_q[b], p = pos[t], keep = taps - 1;
  const int QK = 2 * G * D, C = QK + H * Dv;
  const float* ts = tail + (size_t)min(max(sslots[b], 0), nslots - 1) * keep * C;
  if (blockIdx.y == 0)
    for (int h = lane; h < H; h += 64) {
      const float* z = gz + (size_t)t * 2 * H;
      tok[((size_t)t * H + h) * 2] = expf(a_neg[h] * dr_softplus(z[H + h] + dt_bias[h]));
      tok[((size_t)t * H + h) * 2 + 1] = sigmoid_f(z[h]);
    }
  const float qscale = 1.f / sqrtf((float)D);
  const int lpg = D / 8;                              // lanes per head
  for (int c = 8 * (blockIdx.y * 64 + lane); c - 8 * lane < C; c += 8 * 64 * gridDim.y) {
    const bool ok = c < C;                            // whole waves stay in the loop for the sums
    float acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = 0.f;
    if (ok)
      for (int j = 0; j < taps; ++j) {
        const int s = keep - j;                       // how many tokens back this tap reads
        if (p - s < 0) continue;                      // before the sequence's start
        float f[8];
        if (i - s >= 0) {
          unpack8(*reinterpret_cast<const uint4*>(u + (size_t)(t - s) * ldu + c), f);
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
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      acc[k] = silu_f(acc[k]);
      ss += acc[k] * acc[k];
    }
    ss = dr_group_sum(ss, lpg);                       // q / k heads start on multiples of D
    float mul = 1.f;
    if (c < QK) mul = (c < G * D ? qscale : 1.f) / sqrtf(ss + 1e-6f);
    if (ok) {
      float* o = act + (size_t)t * C + c;
      *reinterpret_cast<float4*>(o) =
          make_float4(acc[0] * mul, acc[1] * mul, acc[2] * mul, acc[3] * mul);
      *reinterpret_cast<float4*>(o + 4) =
          make_float4(acc[4] * mul, acc[5] * mul, acc[6] * mul, acc[7] * mul);
    }
  }
}

template <int MAXD, int TC, int EC, int LPC>   // LPC lanes per column, D <= LPC * MAXD
__global__ __launch_bounds__(EC * LPC) void delta_scan_kernel(
    const float* __restrict__ act, long ld, int H, int D, int Dv, int q_off, int k_off, int v_off,
    int hpg, float* __restrict__ state, const int* __restrict__ state_slots,
    const int* __restrict__ cu_q, const int* __restrict__ positions, const float* __restrict__ tok,
    float* __restrict__ o) {
  constexpr int NTH = EC * LPC;
  constexpr int DPAD = LPC * MAXD;            // padded row length in LDS
  constexpr int NPT = TC * DPAD / NTH;          // staged q (and k) values per thread
  constexpr int NVT = (TC * EC + NTH - 1) / NTH;
  __shared__ __attribute__((aligned(16))) float qs[TC * DPAD];
  __shared__ __attribute__((aligned(16))) float ks[TC * DPAD];
  __shared__ float vs[TC * EC];
  __shared__ float os[TC * EC];
  __shared__ float gs[TC], bs[TC], cs[TC];
  const int b = blockIdx.x, h = blockIdx.y, e0 = blockIdx.z * EC;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (q1 <= q0) return;
  const int tid = threadIdx.x;
  const int dp = tid % LPC, e = tid / LPC;
  const bool col = e0 + e < Dv;
  // a column's rows side by side: state [slots, H, Dv, D]
  float* Sg = state + (((size_t)state_slots[b] * H + h) * Dv + e0 + e) * D + dp * MAXD;
  const bool fresh = positions[q0] == 0;
  float S[MAXD];
  if (!fresh && col && D % 4 == 0) {
#pragma unroll
    for (int i = 0; i < MAXD / 4; ++i) {
      float4 s4 = make_float4(0.f, 0.f, 0.f, 0.f);
      if (dp * MAXD + 4 * i < D) s4 = *reinterpret_cast<const float4*>(Sg + 4 * i);
      S[4 * i] = s4.x; S[4 * i + 1] = s4.y; S[4 * i + 2] = s4.z; S[4 * i + 3] = s4.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < MAXD; ++i)
      S[i] = (!fresh && col && dp * MAXD + i < D) ? Sg[i] : 0.f;
  }
  const size_t qoff = (size_t)q_off + (size_t)(h / hpg) * D;
  const size_t koff = (size_t)k_off + (size_t)(h / hpg) * D;
  const size_t voff = (size_t)v_off + (size_t)h * Dv + e0;
  float rq[NPT], rk[NPT], rv[NVT], rg = 1.f, rb = 0.f;
  auto fetch = [&](int t0) {               // the values of tokens t0 .. t0 + TC into registers
    if (tid < TC) {
      const bool ok = t0 + tid < q1;
      rg = ok ? tok[((size_t)(t0 + tid) * H + h) * 2] : 1.f;
      rb = ok ? tok[((size_t)(t0 + tid) * H + h) * 2 + 1] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
      const int i = tid + NTH * j, tt = i / DPAD, d = i % DPAD;
      const bool ok = t0 + tt < q1 && d < D;
      const float* row = act + (size_t)(ok ? t0 + tt : q0) * ld;
      rq[j] = ok ? row[qoff + d] : 0.f;
      rk[j] = ok ? row[koff + d] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NVT; ++j) {
      const int i = tid + NTH * j, tt = i / EC, c = i % EC;
      const bool ok = i < TC * EC && t0 + tt < q1 && e0 + c < Dv;
      rv[j] = ok ? act[(size_t)(t0 + tt) * ld + voff + c] : 0.f;
    }
  };
  fetch(q0);
  for (int t0 = q0; t0 < q1; t0 += TC) {
    const int nt = min(TC, q1 - t0);
    __syncthreads();                       // the previous group's LDS is consumed
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
      qs[tid + NTH * j] = rq[j];
      ks[tid + NTH * j] = rk[j];
    }
#pragma unroll
    for (int j = 0; j < NVT; ++j)
      if (tid + NTH * j < TC * EC) vs[tid + NTH * j] = rv[j];
    if (tid < TC) { gs[tid] = rg; bs[tid] = rb; }
    __syncthreads();
    if (t0 + TC < q1) fetch(t0 + TC);      // in flight while this group is computed
    // k . q of every token of the group once for all columns; the decayed
    // state is formed while the 16-lane sum of S^T k is under way, so that
    // one multiply-add per row follows the sum
    for (int i = tid; i < TC * LPC; i += NTH) {
      const int tt = i / LPC, pp = i % LPC;
      float c = 0.f;
#pragma unroll
      for (int j = 0; j < MAXD; ++j)
        c += ks[tt * DPAD + pp * MAXD + j] * qs[tt * DPAD + pp * MAXD + j];
      c = dr_lane_sum<LPC>(c);
      if (pp == 0) cs[tt] = c;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      float4 kc[MAXD / 4], qc[MAXD / 4];
      const float4* k4 = reinterpret_cast<const float4*>(ks + tt * DPAD + dp * MAXD);
      const float4* q4 = reinterpret_cast<const float4*>(qs + tt * DPAD + dp * MAXD);
#pragma unroll
      for (int i = 0; i < MAXD / 4; ++i) { kc[i] = k4[i]; qc[i] = q4[i]; }
      const float g = gs[tt], bt = bs[tt], vv = vs[tt * EC + e], kq = cs[tt];
      float r0 = 0.f, r1 = 0.f, s0 = 0.f, s1 = 0.f;
#pragma unroll
      for (int i = 0; i < MAXD / 4; ++i) {
        r0 += S[4 * i] * kc[i].x;     r1 += S[4 * i + 1] * kc[i].y;
        r0 += S[4 * i + 2] * kc[i].z; r1 += S[4 * i + 3] * kc[i].w;
      }
      // the decayed state and the second product are formed while the lane sum
      // of the first is under way
#pragma unroll
      for (int i = 0; i < MAXD / 4; ++i) {
        s0 += S[4 * i] * qc[i].x;     s1 += S[4 * i + 1] * qc[i].y;
        s0 += S[4 * i + 2] * qc[i].z; s1 += S[4 * i + 3] * qc[i].w;
      }
      const float r = dr_lane_sum<LPC>(r0 + r1);
#pragma unroll
      for (int i = 0; i < MAXD; ++i) S[i] *= g;
      const float uu = bt * (vv - g * r);
#pragma unroll
      for (int i = 0; i < MAXD / 4; ++i) {
        S[4 * i] += kc[i].x * uu;     S[4 * i + 1] += kc[i].y * uu;
        S[4 * i + 2] += kc[i].z * uu; S[4 * i + 3] += kc[i].w * uu;
      }
      const float sq = dr_lane_sum<LPC>(s0 + s1);
      if (dp == 0) os[tt * EC + e] = g * sq + uu * kq;
    }
    __syncthreads();
    for (int i = tid; i < nt * EC; i += NTH) {
      const int tt = i / EC, c = i % EC;
      if (e0 + c < Dv) o[(size_t)(t0 + tt) * H * Dv + (size_t)h * Dv + e0 + c] = os[i];
    }
  }
  if (col && D % 4 == 0) {
#pragma unroll
    for (int i = 0; i < MAXD / 4; ++i)
      if (dp * MAXD + 4 * i < D)
        *reinterpret_cast<float4*>(Sg + 4 * i) =
            make_float4(S[4 * i], S[4 * i + 1], S[4 * i + 2], S[4 * i + 3]);
  } else if (col) {
#pragma unroll
    for (int i = 0; i < MAXD; ++i)
      if (dp * MAXD + i < D) Sg[i] = S[i];
  }
}

extern "C" int loqa_delta_prep(const void* u, int u_dt, long ldu, const void* gz, int G, int D,
                               int H, int Dv, const void* cw, int taps, const void* tail,
                               int nslots, const void* a_neg, const void* dt_bias,
                               const void* sslots, const void* cu_q, const void* pos, int B, int T,
                               void* act, void* tok, hipStream_t st) {
  if (T <= 0) return 0;
  if (B <= 0 || taps < 1 || nslots <= 0 || G <= 0 || D <= 0 || D > 512 || H <= 0 || Dv <= 0)
    return (int)hipErrorInvalidValue;
  const int C = 2 * G * D + H * Dv, lpg = D / 8;
  if (u_dt == 0 && D % 8 == 0 && lpg <= 64 && (lpg & (lpg - 1)) == 0 && C % 8 == 0 &&
      ldu % 8 == 0 && ((size_t)u & 15) == 0) {
    const int per = (C + 511) / 512;
    hipLaunchKernelGGL(delta_prep_v8_kernel, dim3(T, T >= 2048 ? (per + 1) / 2 : per), dim3(64), 0,
                       st, (const bf16_t*)u, ldu, (const float*)gz, G, D, H, Dv, (const float*)cw,
                       taps, (const float*)tail, nslots, (const float*)a_neg,
                       (const float*)dt_bias, (const int*)sslots, (const int*)cu_q,
                       (const int*)pos, B, (float*)act, (float*)tok);
    return (int)hipGetLastError();
  }
  const int units = (C + D - 1) / D;
  // many rows: a wave walks several runs
  const dim3 grid(T, T >= 4096 ? (units + 3) / 4 : units);
#define GO(TU)                                                                                   \
  hipLaunchKernelGGL(delta_prep_kernel<TU>, grid, dim3(64), 0, st, (const TU*)u, ldu,            \
                     (const float*)gz, G, D, H, Dv, (const float*)cw, taps, (const float*)tail,  \
                     nslots, (const float*)a_neg, (const float*)dt_bias, (const int*)sslots,     \
                     (const int*)cu_q, (const int*)pos, B, (float*)act, (float*)tok)
  if (u_dt == 0) GO(bf16_t); else GO(float);
#undef GO
  return (int)hipGetLastError();
}

// act: f32 [T, ld]; head h reads q at q_off + (h / hpg) D, k at k_off + (h / hpg) D,
// v at v_off + h Dv; tok [T, H, 2] = (decay, beta); state [slots, H, Dv, D].
extern "C" int loqa_delta_scan(const void* act, long ld, int H, int D, int Dv, int q_off, int k_off,
                               int v_off, int hpg, void* state, int nslots,
                               const void* state_slots, const void* cu_q, const void* positions,
                               const void* tok, void* o, int B, int T, hipStream_t st) {
  if (T <= 0 || B <= 0) return 0;
  if (D > DR_DP * 16 || D <= 0 || Dv <= 0 || hpg <= 0 || H % hpg || !tok)
    return (int)hipErrorInvalidValue;
  (void)nslots;
  // column block: 16 columns (4 waves) share the staged q and k rows. A lone
  // prompt is bound by the latency of a token step, not by the number of
  // compute units it covers, so narrower blocks only stage the same rows more
  // often (measured side by side on a 2048-token prompt, 16 heads x 128
  // columns: 648 us with 8 columns, 549 us with 16, 586 us with 32) - and the
  // denser grid leaves compute units to whatever runs on the other stream.
  const int ec = Dv > 8 ? 16 : (Dv > 4 ? 8 : 4);
#define GOL(MD, TCC, ECC, LL)                                                                     \
  hipLaunchKernelGGL((delta_scan_kernel<MD, TCC, ECC, LL>), dim3(B, H, (Dv + ECC - 1) / ECC),     \
                     dim3(ECC * LL), 0, st, (const float*)act, ld, H, D, Dv, q_off, k_off,        \
                     v_off, hpg, (float*)state, (const int*)state_slots, (const int*)cu_q,        \
                     (const int*)positions, (const float*)tok, (float*)o)
#define GO(MD, TCC, ECC) GOL(MD, TCC, ECC, 16)
#define GOE(MD, TCC)                                                                              \
  do {                                                                                            \
    if (ec == 16) GO(MD, TCC, 16); else if (ec == 8) GO(MD, TCC, 8); else GO(MD, TCC, 4);         \
  } while (0)
  // more than 64 rows: 32 lanes per column (measured on the same prompt: 553 us
  // with 16 lanes x 8 rows, 501 us with 32 lanes x 4 rows)
  if (D <= 64) GOE(4, 16);
  else if (ec == 16 && D <= 128) GOL(4, 16, 16, 32);
  else if (ec == 16) GOL(8, 16, 16, 32);
  else if (D <= 128) GOE(8, 16);
  else GOE(16, 8);
#undef GOE
#undef GO
#undef GOL
  return (int)hipGetLastError();
}

// Mixture-of-experts feed-forward: grouped top-k router, device-side grouping
// of tokens by expert, grouped expert GEMMs, weighted combine.
//
// moe_route_kernel (one wave per token): scores = softmax(z) over all router
//   outputs; choice = score + correction; router outputs form `groups` equal
//   groups of neighbours, a group ranks by its best choice score and only the
//   `keep` best groups stay eligible (the others count as -inf); the `top`
//   best eligible choices are taken; the weights are the plain scores. Mode 1:
//   the choice is by the logit itself (+ bias) and the weights are the softmax
//   over the chosen logits only. Mode 2: scores = sigmoid(z) instead of the
//   softmax. With `grank` n > 1 a group ranks by the sum of its n best choice
//   scores.
// moe_plan_kernel (one workgroup): (token, k) pairs bucketed by expert without
//   a host round trip: offsets[E + 2], perm[P] (pair ids in expert order; the
//   identity bucket E last), pos[P] (where each pair sits).
// moe_grouped_gemm_kernel: C = A . W_e^T per expert segment, 64 x 64 tiles,
//   f32 accumulation over K in ascending order for every output element (so a
//   pair's result does not depend on which other pairs share its tile). Mode
//   1 gathers A rows by token and applies the SwiGLU epilogue to the (gate,
//   up) weight row pairs; mode 2 gathers A rows by token and squares the relu
//   of a single (up) weight set; mode 0 reads the sorted activation rows.
// moe_combine_kernel: out[t] = sum_k weight * (expert output | the input
//   itself for an identity expert), f32.
#include "seqmix.h"

#define MOE_MAX_E 1024

__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, 64);
    const int oi = __shfl_xor(i, o, 64);
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
  }
}

__global__ __launch_bounds__(64) void moe_route_kernel(
    const float* __restrict__ z, const float* __restrict__ corr, const float* __restrict__ bias,
    int mode, int E, int G, int keep, int grank, int top, int* __restrict__ idx,
    float* __restrict__ wt) {
  const int top_softmax = mode == 1;
  __shared__ float sc[MOE_MAX_E], ch[MOE_MAX_E], gs[MOE_MAX_E];
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* zr = z + (size_t)t * E;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) {
    const float v = bias ? zr[e] + bias[e] : zr[e];
    gs[e] = v;                                  // the logit with its bias
    mx = fmaxf(mx, v);
  }
  mx = wave_max(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += 64) {
    const float v = mode == 2 ? sigmoid_f(gs[e]) : expf(gs[e] - mx);
    sc[e] = v;
    sum += v;
  }
  sum = wave_sum(sum);
  const float inv = mode == 2 ? 1.f : 1.f / sum;
  for (int e = lane; e < E; e += 64) {
    if (top_softmax) { ch[e] = gs[e]; continue; }      // scores stay unnormalised: see below
    const float s = sc[e] * inv;
    sc[e] = s;
    ch[e] = corr ? s + corr[e] : s;
  }
  __syncthreads();
  if (G > 1 && keep < G) {
    const int per = E / G;
    for (int g = lane; g < G; g += 64) {
      float b = -INFINITY;
      if (grank <= 1) {
        for (int j = 0; j < per; ++j) b = fmaxf(b, ch[g * per + j]);
      } else {
        // the sum of the group's n best: n passes, each taking the largest entry
        // below the previous one (by value, then index)
        float pv = INFINITY;
        int pi = -1;
        b = 0.f;
        for (int n = 0; n < min(grank, per); ++n) {
          float bv = -INFINITY;
          int bi = -1;
          for (int j = 0; j < per; ++j) {
            const float v = ch[g * per + j];
            const bool below = v < pv || (v == pv && j > pi);
            if (below && (bi < 0 || v > bv)) { bv = v; bi = j; }
          }
          if (bi < 0) break;
          b += bv;
          pv = bv;
          pi = bi;
        }
      }
      gs[g] = b;
    }
    __syncthreads();
    // the `keep` best groups are marked with +inf, then the rest is masked
    for (int k = 0; k < keep; ++k) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int g = lane; g < G; g += 64) {
        const float v = gs[g];
        if (v != INFINITY && (v > bv || bi == 0x7fffffff)) { bv = v; bi = g; }
      }
      wave_argmax(bv, bi);
      if (lane == 0 && bi < G) gs[bi] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < E; e += 64)
      if (gs[e / per] != INFINITY) ch[e] = -INFINITY;
    __syncthreads();
  }
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = ch[e];
      if (v != INFINITY && (v > bv || bi == 0x7fffffff)) { bv = v; bi = e; }
    }
    wave_argmax(bv, bi);
    bi = min(max(bi, 0), E - 1);
    if (lane == 0) {
      idx[(size_t)t * top + k] = bi;
      wt[(size_t)t * top + k] = sc[bi];
      ch[bi] = INFINITY;                      // taken
    }
    __syncthreads();
  }
  if (top_softmax && lane == 0) {
    // softmax over the chosen logits: exp(z - max) of the chosen ones over their sum
    float tot = 0.f;
    for (int k = 0; k < top; ++k) tot += wt[(size_t)t * top + k];
    const float r = 1.f / tot;
    for (int k = 0; k < top; ++k) wt[(size_t)t * top + k] *= r;
  }
}

__global__ __launch_bounds__(256) void moe_plan_kernel(const int* __restrict__ idx, int P, int E,
                                                       int* __restrict__ plan) {
  __shared__ int cnt[MOE_MAX_E + 2];
  int* offsets = plan;                // [E + 2]
  int* perm = plan + E + 2;           // [P]
  int* pos = perm + P;                // [P]
  for (int e = threadIdx.x; e < E + 2; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = min(max(idx[p], 0), E);     // identity experts share bucket E
    atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e <= E; ++e) {
      const int c = cnt[e];
      offsets[e] = run;
      cnt[e] = run;                           // becomes the fill cursor
      run += c;
    }
    offsets[E + 1] = run;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = min(max(idx[p], 0), E);
    const int s = atomicAdd(&cnt[e], 1);
    perm[s] = p;
    pos[p] = s;
  }
}

#define GG_T 64
#define GG_K 16

__device__ __forceinline__ float relu2_f(float z) { const float r = fmaxf(z, 0.f); return r * r; }

template <typename T, int MODE>
__global__ __launch_bounds__(256) void moe_grouped_gemm_kernel(
    const T* __restrict__ A, const T* __restrict__ Wt, const int* __restrict__ plan, int P, int E,
    int top, int K, int N, T* __restrict__ out) {
  constexpr int SWIGLU = MODE == 1;
  constexpr bool GATHER = MODE != 0;
  __shared__ float As[GG_K][GG_T + 1], Bs[GG_K][GG_T + 1], Bu[SWIGLU ? GG_K : 1][GG_T + 1];
  const int* offsets = plan;
  const int* perm = plan + E + 2;
  // which expert segment and which 64-row tile of it this workgroup owns
  int tile = blockIdx.x, e = 0, r0 = 0, r1 = 0;
  for (; e < E; ++e) {
    const int s0 = offsets[e], s1 = offsets[e + 1];
    const int nt = (s1 - s0 + GG_T - 1) / GG_T;
    if (tile < nt) { r0 = s0 + tile * GG_T; r1 = min(s1, r0 + GG_T); break; }
    tile -= nt;
  }
  if (e == E) return;
  const int n0 = blockIdx.y * GG_T;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int wrows = SWIGLU ? 2 * N : N;        // rows of one expert's weight
  const T* We = Wt + (size_t)e * wrows * K;
  float acc[4][4], accu[SWIGLU ? 4 : 1][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) { acc[i][j] = 0.f; if (SWIGLU) accu[i][j] = 0.f; }
  for (int k0 = 0; k0 < K; k0 += GG_K) {
    __syncthreads();
    for (int i = threadIdx.x; i < GG_T * GG_K; i += 256) {
      const int r = i / GG_K, kk = i % GG_K;
      float a = 0.f, b = 0.f, u = 0.f;
      if (k0 + kk < K) {
        if (r0 + r < r1) {
          const size_t src = GATHER ? (size_t)(perm[r0 + r] / top) : (size_t)(r0 + r);
          a = Act<T>::ld(A + src * K + k0 + kk);
        }
        if (n0 + r < N) {
          b = Act<T>::ld(We + (size_t)(n0 + r) * K + k0 + kk);
          if (SWIGLU) u = Act<T>::ld(We + (size_t)(N + n0 + r) * K + k0 + kk);
        }
      }
      As[kk][r] = a;
      Bs[kk][r] = b;
      if (SWIGLU) Bu[kk][r] = u;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GG_K; ++kk) {
      float a[4], b[4], u[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] = As[kk][ty * 4 + i];
        b[i] = Bs[kk][tx * 4 + i];
        if (SWIGLU) u[i] = Bu[kk][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] += a[i] * b[j];
          if (SWIGLU) accu[i][j] += a[i] * u[j];
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + ty * 4 + i;
    if (r >= r1) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N)
        Act<T>::st(out + (size_t)r * N + n, SWIGLU ? silu_f(acc[i][j]) * accu[i][j]
                                                   : MODE == 2 ? relu2_f(acc[i][j]) : acc[i][j]);
    }
  }
}

// The bf16 path of the grouped GEMM on the matrix cores (K a multiple of 32):
// v_mfma_f32_16x16x32_bf16 with the expert's weight rows as the A operand and
// the (gathered) token rows as B, both fragments loaded straight from global
// memory as one 16-byte load per lane (weights are [n][k] and rows [m][k], so a
// lane's 8 k-values are contiguous). A workgroup owns 64 token rows x 64
// features of one expert segment; each of its 4 waves takes 16 features (and
// the 16 matching up-rows for SwiGLU) against all 64 rows, so the row fragments
// are shared through L1. An accumulator lane holds 4 consecutive features of
// one token row. Per output element the sum over K has a fixed order.
template <int MODE>
__global__ __launch_bounds__(256) void moe_grouped_gemm_mfma_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Wt, const int* __restrict__ plan, int P,
    int E, int top, int K, int N, bf16_t* __restrict__ out) {
  constexpr int SWIGLU = MODE == 1;
  constexpr bool GATHER = MODE != 0;
  const int* offsets = plan;
  const int* perm = plan + E + 2;
  int tile = blockIdx.x, e = 0, r0 = 0, r1 = 0;
  for (; e < E; ++e) {
    const int s0 = offsets[e], s1 = offsets[e + 1];
    const int nt = (s1 - s0 + GG_T - 1) / GG_T;
    if (tile < nt) { r0 = s0 + tile * GG_T; r1 = min(s1, r0 + GG_T); break; }
    tile -= nt;
  }
  if (e == E) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int fr = lane & 15, fq = lane >> 4;
  const int nb = blockIdx.y * GG_T + wave * 16;         // this wave's 16 features
  if (nb >= N) return;
  const int wrows = SWIGLU ? 2 * N : N;
  const bf16_t* We = Wt + (size_t)e * wrows * K;
  const int nrow = min(nb + fr, N - 1);                 // clamped: loads stay in range
  const bf16_t* wg = We + (size_t)nrow * K + fq * 8;
  const bf16_t* wu = SWIGLU ? We + (size_t)(N + nrow) * K + fq * 8 : nullptr;
  const bf16_t* arow[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = min(r0 + 16 * j + fr, r1 - 1);
    const size_t src = GATHER ? (size_t)(perm[r] / top) : (size_t)r;
    arow[j] = A + src * K + fq * 8;
  }
  float4v acc[4], accu[SWIGLU ? 4 : 1];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    acc[j] = float4v{0.f, 0.f, 0.f, 0.f};
    if (SWIGLU) accu[j] = float4v{0.f, 0.f, 0.f, 0.f};
  }
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bf16x8 a = *reinterpret_cast<const bf16x8*>(wg + k0);
    bf16x8 au;
    if (SWIGLU) au = *reinterpret_cast<const bf16x8*>(wu + k0);
    bf16x8 b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j] = *reinterpret_cast<const bf16x8*>(arow[j] + k0);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[j], acc[j], 0, 0, 0);
      if (SWIGLU) accu[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(au, b[j], accu[j], 0, 0, 0);
    }
  }
  // acc[j][i]: feature nb + 4 fq + i of token row r0 + 16 j + fr
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = r0 + 16 * j + fr;
    if (r >= r1) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = nb + 4 * fq + i;
      if (n < N) {
        const float v = SWIGLU ? silu_f(acc[j][i]) * accu[j][i]
                               : MODE == 2 ? relu2_f(acc[j][i]) : acc[j][i];
        out[(size_t)r * N + n] = f2bf(v);
      }
    }
  }
}

// Prompt-sized batches (hundreds of rows per expert): 128 token rows x 128
// features per workgroup, the token rows of a 64-wide K chunk staged once in
// LDS for the 4 waves (the next chunk's rows already in flight in registers),
// weights streamed straight from global memory. A wave owns 2 feature
// sub-tiles of 16 (and their up-rows for SwiGLU): every weight fragment is
// loaded once per workgroup and feeds 8 MFMAs, every staged row fragment read
// from LDS feeds 2 (4 with SwiGLU). Same fragment layout and summation order
// as the kernel above.
#define GG_R2 128
#define GG_KC 64
#define GG_NF 2

template <int MODE>
__global__ __launch_bounds__(256) void moe_grouped_gemm_mfma2_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Wt, const int* __restrict__ plan, int P,
    int E, int top, int K, int N, bf16_t* __restrict__ out) {
  constexpr int SWIGLU = MODE == 1;
  constexpr bool GATHER = MODE != 0;
  __shared__ __attribute__((aligned(16))) bf16_t rows[GG_R2][GG_KC + 8];
  const int* offsets = plan;
  const int* perm = plan + E + 2;
  int tile = blockIdx.x, e = 0, r0 = 0, r1 = 0;
  for (; e < E; ++e) {
    const int s0 = offsets[e], s1 = offsets[e + 1];
    const int nt = (s1 - s0 + GG_R2 - 1) / GG_R2;
    if (tile < nt) { r0 = s0 + tile * GG_R2; r1 = min(s1, r0 + GG_R2); break; }
    tile -= nt;
  }
  if (e == E) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int fr = lane & 15, fq = lane >> 4;
  const int nb = blockIdx.y * (64 * GG_NF) + wave * (16 * GG_NF);
  const bool wave_on = nb < N;                           // idle waves still stage rows
  const int wrows = SWIGLU ? 2 * N : N;
  const bf16_t* We = Wt + (size_t)e * wrows * K;
  const bf16_t* wg[GG_NF];
  const bf16_t* wu[GG_NF];
#pragma unroll
  for (int f = 0; f < GG_NF; ++f) {
    const int nrow = min(nb + 16 * f + fr, N - 1);
    wg[f] = We + (size_t)nrow * K + fq * 8;
    wu[f] = SWIGLU ? We + (size_t)(N + nrow) * K + fq * 8 : nullptr;
  }
  // staging: thread -> 4 chunks of 8 entries: row = (tid + 256 j) / 8, column chunk = % 8
  const bf16_t* srow[4];
  int srr[4], scc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = threadIdx.x + 256 * j;
    srr[j] = i >> 3;
    scc[j] = (i & 7) * 8;
    const int r = min(r0 + srr[j], r1 - 1);
    const size_t src = GATHER ? (size_t)(perm[r] / top) : (size_t)r;
    srow[j] = A + src * K + scc[j];
  }
  float4v acc[GG_NF][8], accu[SWIGLU ? GG_NF : 1][SWIGLU ? 8 : 1];
#pragma unroll
  for (int f = 0; f < GG_NF; ++f)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      acc[f][j] = float4v{0.f, 0.f, 0.f, 0.f};
      if (SWIGLU) accu[f][j] = float4v{0.f, 0.f, 0.f, 0.f};
    }
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  u32x4 pre[4];                                  // (a plain vector type: stays in registers)
#pragma unroll
  for (int j = 0; j < 4; ++j) pre[j] = *reinterpret_cast<const u32x4*>(srow[j]);
  // this chunk's weight fragments (2 k-steps); the next chunk's are requested
  // before this chunk's MFMAs, so the weight stream's latency stays hidden
  bf16x8 wa[2][GG_NF], wb[SWIGLU ? 2 : 1][GG_NF];
#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int f = 0; f < GG_NF; ++f) {
      wa[q][f] = *reinterpret_cast<const bf16x8*>(wg[f] + 32 * q);
      if (SWIGLU) wb[q][f] = *reinterpret_cast<const bf16x8*>(wu[f] + 32 * q);
    }
  for (int k0 = 0; k0 < K; k0 += GG_KC) {
    __syncthreads();                                     // the previous chunk is consumed
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4*>(&rows[srr[j]][scc[j]]) = pre[j];
    __syncthreads();
    const bool more = k0 + GG_KC < K;
    bf16x8 na[2][GG_NF], nb2[SWIGLU ? 2 : 1][GG_NF];
    if (more) {
#pragma unroll
      for (int j = 0; j < 4; ++j) pre[j] = *reinterpret_cast<const u32x4*>(srow[j] + k0 + GG_KC);
#pragma unroll
      for (int q = 0; q < 2; ++q)
#pragma unroll
        for (int f = 0; f < GG_NF; ++f) {
          na[q][f] = *reinterpret_cast<const bf16x8*>(wg[f] + k0 + GG_KC + 32 * q);
          if (SWIGLU) nb2[q][f] = *reinterpret_cast<const bf16x8*>(wu[f] + k0 + GG_KC + 32 * q);
        }
    }
    if (wave_on) {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const bf16x8 b = *reinterpret_cast<const bf16x8*>(&rows[16 * j + fr][32 * q + fq * 8]);
#pragma unroll
          for (int f = 0; f < GG_NF; ++f) {
            acc[f][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[q][f], b, acc[f][j], 0, 0, 0);
            if (SWIGLU)
              accu[f][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[q][f], b, accu[f][j], 0, 0, 0);
          }
        }
      }
    }
    if (more) {
#pragma unroll
      for (int q = 0; q < 2; ++q)
#pragma unroll
        for (int f = 0; f < GG_NF; ++f) {
          wa[q][f] = na[q][f];
          if (SWIGLU) wb[q][f] = nb2[q][f];
        }
    }
  }
  if (!wave_on) return;
#pragma unroll
  for (int f = 0; f < GG_NF; ++f)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int r = r0 + 16 * j + fr;
      if (r >= r1) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = nb + 16 * f + 4 * fq + i;
        if (n < N) {
          const float v = SWIGLU ? silu_f(acc[f][j][i]) * accu[f][j][i]
                                 : MODE == 2 ? relu2_f(acc[f][j][i]) : acc[f][j][i];
          out[(size_t)r * N + n] = f2bf(v);
        }
      }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    const T* __restrict__ h, const T* __restrict__ y, const int* __restrict__ idx,
    const float* __restrict__ wt, const int* __restrict__ plan, int P, int top, int E, int d,
    float* __restrict__ out) {
  const int t = blockIdx.x;
  const int* pos = plan + E + 2 + P;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < d; c += gridDim.y * blockDim.x) {
    float s = 0.f;
    for (int k = 0; k < top; ++k) {
      const int p = t * top + k;
      const float v = idx[p] >= E ? Act<T>::ld(h + (size_t)t * d + c)
                                  : Act<T>::ld(y + (size_t)pos[p] * d + c);
      s += wt[p] * v;
    }
    out[(size_t)t * d + c] = s;
  }
}

// 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ACT 0: SiLU, 1: the tanh form of GELU
template <typename T, int ACT>
__global__ __launch_bounds__(256) void act_mul_any_kernel(const T* __restrict__ x, int F,
                                                          T* __restrict__ y) {
  const size_t r = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < F; c += gridDim.y * blockDim.x) {
    const float g = Act<T>::ld(x + r * 2 * F + c);
    Act<T>::st(y + r * F + c, (ACT == 1 ? gelu_tanh_f(g) : silu_f(g)) * Act<T>::ld(x + r * 2 * F + F + c));
  }
}

extern "C" int loqa_act_mul_any(const void* x, int dt, int T, int F, int act, void* y,
                                hipStream_t st) {
  if (T <= 0) return 0;
  if (act < 0 || act > 1) return (int)hipErrorInvalidValue;
  const dim3 grid(T, T >= 512 ? 1 : (F + 255) / 256);
#define GO(TT, A)                                                                             \
  hipLaunchKernelGGL((act_mul_any_kernel<TT, A>), grid, dim3(256), 0, st, (const TT*)x, F, (TT*)y)
  if (dt == 0 && act == 0) GO(bf16_t, 0);
  else if (dt == 0) GO(bf16_t, 1);
  else if (act == 0) GO(float, 0);
  else GO(float, 1);
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_moe_route(const void* z, const void* corr, const void* bias, int mode,
                              int E, int G, int keep, int grank, int top, void* idx, void* wt,
                              int T, hipStream_t st) {
  if (T <= 0) return 0;
  if (E > MOE_MAX_E || E <= 0 || G <= 0 || E % G || top <= 0 || top > E || mode < 0 || mode > 2)
    return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(moe_route_kernel, dim3(T), dim3(64), 0, st, (const float*)z, (const float*)corr,
                     (const float*)bias, mode, E, G, keep, grank, top, (int*)idx, (float*)wt);
  return (int)hipGetLastError();
}

extern "C" int loqa_moe_plan(const void* idx, int P, int E, void* plan, hipStream_t st) {
  if (E > MOE_MAX_E) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(256), 0, st, (const int*)idx, P, E, (int*)plan);
  return (int)hipGetLastError();
}

extern "C" int loqa_moe_grouped_gemm(const void* A, int dt, const void* W, const void* plan, int P,
                                     int E, int top, int K, int N, int mode, void* out,
                                     hipStream_t st) {
  if (P <= 0) return 0;
  if (mode < 0 || mode > 2) return (int)hipErrorInvalidValue;
  const dim3 grid((P + GG_T - 1) / GG_T + E, (N + GG_T - 1) / GG_T);
#define BY_MODE(KERNEL, GRID, TT)                                                               \
  do {                                                                                          \
    if (mode == 1)                                                                              \
      hipLaunchKernelGGL(KERNEL(1), GRID, dim3(256), 0, st, (const TT*)A, (const TT*)W,         \
                         (const int*)plan, P, E, top, K, N, (TT*)out);                          \
    else if (mode == 2)                                                                         \
      hipLaunchKernelGGL(KERNEL(2), GRID, dim3(256), 0, st, (const TT*)A, (const TT*)W,         \
                         (const int*)plan, P, E, top, K, N, (TT*)out);                          \
    else                                                                                        \
      hipLaunchKernelGGL(KERNEL(0), GRID, dim3(256), 0, st, (const TT*)A, (const TT*)W,         \
                         (const int*)plan, P, E, top, K, N, (TT*)out);                          \
  } while (0)
#define K_MFMA2(M) (moe_grouped_gemm_mfma2_kernel<M>)
#define K_MFMA(M) (moe_grouped_gemm_mfma_kernel<M>)
#define K_BF16(M) (moe_grouped_gemm_kernel<bf16_t, M>)
#define K_F32(M) (moe_grouped_gemm_kernel<float, M>)
  if (dt == 0 && K % GG_KC == 0 && P >= 16 * (E > 0 ? E : 1) * 4 && P >= 1024) {
    // prompt-sized: on average at least 64 rows per expert
    const dim3 g2((P + GG_R2 - 1) / GG_R2 + E, (N + 64 * GG_NF - 1) / (64 * GG_NF));
    BY_MODE(K_MFMA2, g2, bf16_t);
  } else if (dt == 0 && K >= 32 && K % 32 == 0) {
    BY_MODE(K_MFMA, grid, bf16_t);
  } else if (dt == 0) {
    BY_MODE(K_BF16, grid, bf16_t);
  } else {
    BY_MODE(K_F32, grid, float);
  }
#undef K_MFMA2
#undef K_MFMA
#undef K_BF16
#undef K_F32
#undef BY_MODE
  return (int)hipGetLastError();
}

extern "C" int loqa_moe_combine(const void* h, const void* y, int dt, const void* idx,
                                const void* wt, const void* plan, int T, int top, int E, int d,
                                void* out, hipStream_t st) {
  if (T <= 0) return 0;
  const dim3 cgrid(T, T >= 512 ? 1 : (d + 255) / 256);
  if (dt == 0)
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, cgrid, dim3(256), 0, st, (const bf16_t*)h,
                       (const bf16_t*)y, (const int*)idx, (const float*)wt, (const int*)plan, T * top,
                       top, E, d, (float*)out);
  else
    hipLaunchKernelGGL(moe_combine_kernel<float>, cgrid, dim3(256), 0, st, (const float*)h,
                       (const float*)y, (const int*)idx, (const float*)wt, (const int*)plan, T * top,
                       top, E, d, (float*)out);
  return (int)hipGetLastError();
}

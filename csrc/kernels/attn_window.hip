// Softmax attention over paged K / V with a sliding window, kept first tokens
// and score soft-capping, and the launch that prepares its q / k rows.
//
//   score(i, j) = q_i . k_j * scale;   with cap > 0: cap * tanh(score / cap)
//   key j is visible to the query at position p if j <= p and
//        (window == 0  or  p - j < window  or  j < keep_first)
//   out_i = softmax_j(score) V,  times sigmoid(gate_i) per entry if a gate is given
//
// K pages are [blocks][BLK][G * D], V pages [blocks][BLK][G * Dv]; query head h
// reads key/value head h / (H / G). Rows find their sequence through cu_q and
// their keys through the block table, so prompt portions, decode tokens and
// mixed batches are one launch. window = 0 with cap = 0 is plain causal
// attention.
//
// qk_prep_append_kernel (one workgroup per token, a wave per head): the first
// `dims` entries of each q and k head rotate pairwise (2i with 2i + 1) by the
// position's angles, each head is divided by its root mean square (no weight),
// q is multiplied by the position's temperature; q out, k into its page, and
// the value row (its own projection columns, or the k columns as projected)
// into its page. Statistics, angles and temperature are f32.
//
// window_attn_keys_kernel (any dtype, any head size up to 512; decode steps,
// short feeds and the exact f32 mode): a workgroup per (token, key/value head)
// serves REP query heads of the group at once, so K and V are read once per
// group. The visible keys go in 64-key windows aligned to multiples of 64
// positions, one per wave in turn (window index modulo the wave count): scores
// with a lane per key, an online softmax per head across the wave, values with
// a lane per output column. The waves' partial (max, sum, accumulator) triples
// merge through LDS in wave order. Which windows a wave takes and the order of
// every sum depend only on the query's position, never on the batch.
//
// window_attn_mfma_kernel (bf16, D and Dv in {64, 128}; prompt portions): a
// workgroup per (128 query rows of one sequence, query head); each wave owns 32
// rows. K and V tiles of 64 keys are gathered from the pages into LDS for all
// waves (the next tile's 16-byte chunks already in flight in registers);
// S^T = K Q^T and O^T += V^T P^T run on v_mfma_f32_32x32x16_bf16 with the query
// on the MFMA lane, so the online softmax is in-register. Tiles that lie wholly
// between the kept first tokens and the rows' windows are skipped.
#include "seqmix.h"

#define WA_NW 4                      // waves of the keys form

struct WinAttnParams {
  const void* q; const void* kc; const void* vc; int blk; long cache_rows;
  const int* cu_q; const int* ctx; const int* bt; int max_blocks; const int* pos;
  const void* gate; long gate_ld; float scale, cap; int window, keep_first;
  int B, T, H, G, D, Dv; void* o;
};

__device__ __forceinline__ int wa_seq_of_row(const int* __restrict__ cu_q, int B, int t) {
  int b = 0;
  while (b + 1 < B && t >= cu_q[b + 1]) ++b;
  return b;
}

// ------------------------------------------------------------------ q / k rows
template <typename T>
__global__ __launch_bounds__(256) void qk_prep_append_kernel(
    const T* __restrict__ u, long ldu, int H, int G, int D, int Dv, int v_off,
    const float* __restrict__ cs, int max_pos, int dims, float eps, float coef, int every,
    const int* __restrict__ pos, T* __restrict__ kc, T* __restrict__ vc, long cache_rows,
    const int* __restrict__ kvslots, T* __restrict__ q) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int p = pos[t];
  const long slot = kvslots[t];
  const bool store = slot >= 0 && slot < cache_rows;
  const T* ur = u + (size_t)t * ldu;
  const float* csr = dims ? cs + (size_t)min(max(p, 0), max_pos - 1) * dims : nullptr;
  const float temp = 1.f + coef * logf((float)((p + 1) / every) + 1.f);
  constexpr int NP = 4;                           // pairs per lane (D <= 512)
  for (int job = wave; job < H + G; job += 4) {
    const bool isq = job < H;
    const T* src = ur + (size_t)job * D;          // q heads, then k heads
    float a[NP], b[NP];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int e = 2 * (lane + 64 * i);
      a[i] = b[i] = 0.f;
      if (e < D) {
        a[i] = Act<T>::ld(src + e);
        b[i] = Act<T>::ld(src + e + 1);
        if (!isq && v_off < 0 && store) {         // the values are the keys as projected
          T* vr = vc + (size_t)slot * G * Dv + (size_t)(job - H) * Dv + e;
          Act<T>::st(vr, a[i]);
          Act<T>::st(vr + 1, b[i]);
        }
        if (e < dims) {
          const float c = csr[e], s = csr[e + 1];
          const float x = a[i] * c - b[i] * s, y = b[i] * c + a[i] * s;
          a[i] = x;
          b[i] = y;
        }
        ss += a[i] * a[i] + b[i] * b[i];
      }
    }
    ss = wave_sum(ss);
    float inv = 1.f / sqrtf(ss / (float)D + eps);
    if (isq) inv *= temp;
    T* dst = isq ? q + (size_t)t * H * D + (size_t)job * D
                 : (store ? kc + (size_t)slot * G * D + (size_t)(job - H) * D : nullptr);
    if (dst) {
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int e = 2 * (lane + 64 * i);
        if (e < D) {
          Act<T>::st(dst + e, a[i] * inv);
          Act<T>::st(dst + e + 1, b[i] * inv);
        }
      }
    }
  }
  if (v_off >= 0 && store) {
    T* vr = vc + (size_t)slot * G * Dv;
    for (int c = threadIdx.x; c < G * Dv; c += blockDim.x) vr[c] = ur[v_off + c];
  }
}

// ------------------------------------------------------------ few rows, many keys
template <typename T> struct WaVec;
template <> struct WaVec<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void ld(const bf16_t* p, float* f) {
    unpack8(*reinterpret_cast<const uint4*>(p), f);
  }
};
template <> struct WaVec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void ld(const float* p, float* f) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
  }
};

template <typename T, int REP, int NV>
__global__ __launch_bounds__(64 * WA_NW) void window_attn_keys_kernel(WinAttnParams p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x, g = blockIdx.y;
  if (t >= p.cu_q[p.B]) return;
  const int b = wa_seq_of_row(p.cu_q, p.B, t);
  const int D = p.D, Dv = p.Dv, rep = p.H / p.G;
  const int r0 = blockIdx.z * REP;                 // first head of the group this block serves
  const int nr = min(REP, rep - r0);
  float* qs = lds;                                 // [REP][D]
  float* ws = qs + REP * D + wave * REP * 64;      // per wave [REP][64]
  for (int i = threadIdx.x; i < nr * D; i += blockDim.x)
    qs[i] = Act<T>::ld((const T*)p.q + (size_t)t * p.H * D + (size_t)(g * rep + r0) * D + i);
  __syncthreads();
  const int pq = p.pos[t];
  const int hi = min(pq, p.ctx[b] - 1);
  const int lo = p.window > 0 ? max(0, pq - p.window + 1) : 0;
  // windows of 64 keys: those that hold kept first tokens, then those from lo on
  const int w_lo = lo >> 6, w_hi = hi >> 6;
  const int n1 = p.window > 0 ? min((min(p.keep_first, lo) + 63) >> 6, w_lo) : 0;
  const int nwin = hi >= 0 ? n1 + (w_hi - w_lo + 1) : 0;
  const int* bt = p.bt + (size_t)b * p.max_blocks;
  const T* kc = (const T*)p.kc;
  const T* vc = (const T*)p.vc;
  const size_t GD = (size_t)p.G * D, GDv = (size_t)p.G * Dv;
  float m[REP], l[REP], acc[REP][NV];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[r][i] = 0.f;
  }
  const bool vec = D % WaVec<T>::N == 0;
  for (int wk = wave; wk < nwin; wk += WA_NW) {
    const int k0 = (wk < n1 ? wk : w_lo + (wk - n1)) << 6;
    const int j = k0 + lane;
    const bool seen = j <= hi && (p.window <= 0 || pq - j < p.window || j < p.keep_first);
    float s[REP];
#pragma unroll
    for (int r = 0; r < REP; ++r) s[r] = 0.f;
    if (seen) {
      const long row = min(max((long)bt[j / p.blk] * p.blk + j % p.blk, 0L), p.cache_rows - 1);
      const T* kr = kc + (size_t)row * GD + (size_t)g * D;
      if (vec) {
        for (int e = 0; e < D; e += WaVec<T>::N) {
          float f[WaVec<T>::N];
          WaVec<T>::ld(kr + e, f);
#pragma unroll
          for (int r = 0; r < REP; ++r)
#pragma unroll
            for (int i = 0; i < WaVec<T>::N; ++i) s[r] += qs[r * D + e + i] * f[i];
        }
      } else {
        for (int e = 0; e < D; ++e) {
          const float f = Act<T>::ld(kr + e);
#pragma unroll
          for (int r = 0; r < REP; ++r) s[r] += qs[r * D + e] * f;
        }
      }
    }
    float alpha[REP];
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      float sv = s[r] * p.scale;
      if (p.cap > 0.f) sv = p.cap * tanhf(sv / p.cap);
      if (!seen) sv = -INFINITY;
      const float mn = fmaxf(m[r], wave_max(sv));      // a window holds at least one visible key
      const float e = seen ? expf(sv - mn) : 0.f;
      alpha[r] = expf(m[r] - mn);
      l[r] = l[r] * alpha[r] + wave_sum(e);
      m[r] = mn;
      ws[r * 64 + lane] = e;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < REP; ++r)
#pragma unroll
      for (int i = 0; i < NV; ++i) acc[r][i] *= alpha[r];
    const int nk = min(64, hi - k0 + 1);
    for (int kk = 0; kk < nk; ++kk) {
      const int jj = k0 + kk;
      const long row = min(max((long)bt[jj / p.blk] * p.blk + jj % p.blk, 0L), p.cache_rows - 1);
      const T* vr = vc + (size_t)row * GDv + (size_t)g * Dv;
      float v[NV];
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int e = lane + 64 * i;
        v[i] = e < Dv ? Act<T>::ld(vr + e) : 0.f;
      }
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        const float w = ws[r * 64 + kk];
#pragma unroll
        for (int i = 0; i < NV; ++i) acc[r][i] += w * v[i];
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  // merge the waves' partials in wave order
  __syncthreads();                                   // qs / ws are free
  float* mm = lds;                                   // [WA_NW][REP]
  float* ll = mm + WA_NW * REP;                      // [WA_NW][REP]
  float* aa = ll + WA_NW * REP;                      // [WA_NW][REP][NV * 64]
  if (lane == 0)
#pragma unroll
    for (int r = 0; r < REP; ++r) { mm[wave * REP + r] = m[r]; ll[wave * REP + r] = l[r]; }
#pragma unroll
  for (int r = 0; r < REP; ++r)
#pragma unroll
    for (int i = 0; i < NV; ++i) aa[((wave * REP + r) * NV + i) * 64 + lane] = acc[r][i];
  __syncthreads();
  for (int idx = threadIdx.x; idx < nr * NV * 64; idx += blockDim.x) {
    const int r = idx / (NV * 64), c = idx % (NV * 64), i = c >> 6, ln = c & 63;
    const int e = ln + 64 * i;
    if (e >= Dv) continue;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < WA_NW; ++w) M = fmaxf(M, mm[w * REP + r]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < WA_NW; ++w) {
      const float mw = mm[w * REP + r];
      const float f = mw == -INFINITY ? 0.f : expf(mw - M);
      num += f * aa[((w * REP + r) * NV + i) * 64 + ln];
      den += f * ll[w * REP + r];
    }
    float out = den > 0.f ? num / den : 0.f;
    const int h = g * rep + r0 + r;
    if (p.gate)
      out *= sigmoid_f(Act<T>::ld((const T*)p.gate + (size_t)t * p.gate_ld + (size_t)h * Dv + e));
    Act<T>::st((T*)p.o + (size_t)t * p.H * Dv + (size_t)h * Dv + e, out);
  }
}

// ------------------------------------------------------------ prompt portions
#define WM_THREADS 256
#define WM_WAVES 4
#define WM_TILE 64

typedef short wm_v4s __attribute__((ext_vector_type(4)));

template <int DK, int DV>
struct WinMfmaSmem {
  bf16_t k[WM_TILE][DK + 8];
  bf16_t v[WM_TILE][DV + 32];
};

// tanh through the hardware's exp2 and reciprocal (for scores that are rounded
// to bfloat16 weights afterwards)
__device__ __forceinline__ float tanh_fast(float z) {
  return 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(2.885390081777927f * z));
}

template <int DK, int DV>
__global__ __launch_bounds__(WM_THREADS) void window_attn_mfma_kernel(WinAttnParams p) {
  __shared__ __attribute__((aligned(16))) WinMfmaSmem<DK, DV> sm;
  constexpr int NS = DK / 16, NDT = DV / 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = lane >> 5;
  const int head = blockIdx.y, b = blockIdx.z;
  const int g = head / (p.H / p.G);
  const int q0 = p.cu_q[b], qlen = p.cu_q[b + 1] - q0;
  // long row blocks (the most keys) start first
  const int nblk = (int)gridDim.x;
  const int row_lo = (nblk - 1 - (int)blockIdx.x) * (WM_WAVES * 32);
  if (row_lo >= qlen) return;
  const int row_hi = min(qlen - 1, row_lo + WM_WAVES * 32 - 1);
  const int klen = p.ctx[b];
  const int qi = row_lo + wave * 32 + (lane & 31);
  const bool valid = qi < qlen;
  const int qpos = p.pos[q0 + (valid ? qi : row_hi)];
  const int pos_lo = p.pos[q0 + row_lo];
  const int kend = min(klen, p.pos[q0 + row_hi] + 1);     // positions grow along a feed
  // key tiles: those holding kept first tokens, then from the first window on
  const int wg_lo = p.window > 0 ? max(0, pos_lo - p.window + 1) : 0;
  const int lo_t = (wg_lo / WM_TILE) * WM_TILE;
  const int n1 = p.window > 0 ? min((min(p.keep_first, wg_lo) + WM_TILE - 1) / WM_TILE, lo_t / WM_TILE) : 0;
  const int ntiles = n1 + (kend - lo_t + WM_TILE - 1) / WM_TILE;
  // this wave's rows: what they can see at all
  const int wrow_lo = min(row_lo + wave * 32, row_hi), wrow_hi = min(row_lo + wave * 32 + 31, row_hi);
  const int wpos_lo = p.pos[q0 + wrow_lo], wpos_hi = p.pos[q0 + wrow_hi];
  const bool wave_rows = row_lo + wave * 32 <= row_hi;

  bf16x8 qf[NS];
  {
    const bf16_t* qrow = (const bf16_t*)p.q + (size_t)(q0 + (valid ? qi : row_hi)) * p.H * DK +
                         (size_t)head * DK;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      uint4 v = valid ? *reinterpret_cast<const uint4*>(qrow + 16 * s + 8 * h) : make_uint4(0, 0, 0, 0);
      qf[s] = *reinterpret_cast<bf16x8*>(&v);
    }
  }
  float16v acc[NDT];
#pragma unroll
  for (int i = 0; i < NDT; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
  float m_run = -1e30f, l_run = 0.f;
  constexpr int CHK = DK / 8, CHV = DV / 8;
  const size_t kst = (size_t)p.G * DK, vst = (size_t)p.G * DV;
  const bf16_t* kbase = (const bf16_t*)p.kc + (size_t)g * DK;
  const bf16_t* vbase = (const bf16_t*)p.vc + (size_t)g * DV;
  const int* bt = p.bt + (size_t)b * p.max_blocks;
  const float scale_log2 = p.scale * 1.4426950408889634f;
  const float cap_log2 = p.cap * 1.4426950408889634f, inv_cap = p.cap > 0.f ? p.scale / p.cap : 0.f;

  // K / V tiles go through registers: the next tile's 16-byte chunks are
  // requested before this tile's math and stored to LDS after it
  constexpr int NKC = WM_TILE * CHK / WM_THREADS, NVC = WM_TILE * CHV / WM_THREADS;
  uint4 pk[NKC], pv[NVC];
  auto page_row = [&](int j) -> size_t {
    return (size_t)min(max((long)bt[j / p.blk] * p.blk + j % p.blk, 0L), p.cache_rows - 1);
  };
  auto fetch = [&](int kt) {
#pragma unroll
    for (int j = 0; j < NKC; ++j) {
      const int c = threadIdx.x + WM_THREADS * j, kr = c / CHK, cc = (c - kr * CHK) * 8;
      pk[j] = kt + kr < kend ? *reinterpret_cast<const uint4*>(kbase + page_row(kt + kr) * kst + cc)
                             : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < NVC; ++j) {
      const int c = threadIdx.x + WM_THREADS * j, kr = c / CHV, cc = (c - kr * CHV) * 8;
      pv[j] = kt + kr < kend ? *reinterpret_cast<const uint4*>(vbase + page_row(kt + kr) * vst + cc)
                             : make_uint4(0, 0, 0, 0);
    }
  };
  auto tile_at = [&](int i) { return i < n1 ? i * WM_TILE : lo_t + (i - n1) * WM_TILE; };
  fetch(tile_at(0));
  for (int ti = 0; ti < ntiles; ++ti) {
    const int kt = tile_at(ti);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NKC; ++j) {
      const int c = threadIdx.x + WM_THREADS * j, kr = c / CHK, cc = (c - kr * CHK) * 8;
      *reinterpret_cast<uint4*>(&sm.k[kr][cc]) = pk[j];
    }
#pragma unroll
    for (int j = 0; j < NVC; ++j) {
      const int c = threadIdx.x + WM_THREADS * j, kr = c / CHV, cc = (c - kr * CHV) * 8;
      *reinterpret_cast<uint4*>(&sm.v[kr][cc]) = pv[j];
    }
    __syncthreads();
    if (ti + 1 < ntiles) fetch(tile_at(ti + 1));
    // a wave whose rows see nothing of this tile only keeps the barriers
    bool sees = wave_rows && kt <= wpos_hi;
    if (sees && p.window > 0 && kt + WM_TILE <= wpos_lo - p.window + 1 && kt >= p.keep_first)
      sees = false;
    if (!sees) continue;

    float16v st[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int j = 0; j < 16; ++j) st[t][j] = 0.f;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(&sm.k[32 * t + (lane & 31)][16 * s + 8 * h]);
        st[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[s], st[t], 0, 0, 0);
      }
    }
    bf16x8 pf[2][2];
    {
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int key = kt + 32 * t + (j & 3) + 8 * (j >> 2) + 4 * h;
          float sv = p.cap > 0.f ? cap_log2 * tanh_fast(st[t][j] * inv_cap) : st[t][j] * scale_log2;
          if (key >= kend || key > qpos ||
              (p.window > 0 && qpos - key >= p.window && key >= p.keep_first))
            sv = -INFINITY;
          st[t][j] = sv;
          mx = fmaxf(mx, sv);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      const float alpha = exp2f(m_run - m_new);
      float ls = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float e = exp2f(st[t][8 * s2 + j] - m_new);
            ls += e;
            pf[t][s2][j] = (__bf16)e;
          }
      ls += __shfl_xor(ls, 32, 64);
      l_run = l_run * alpha + ls;
      m_run = m_new;
#pragma unroll
      for (int i = 0; i < NDT; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] *= alpha;
    }
    const int g4 = lane >> 4, li = lane & 15;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const int c0 = 32 * dt + 16 * (g4 & 1) + 4 * (li & 3);
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const int kb = 32 * t + 16 * s2 + 4 * h + (li >> 2);
          const wm_v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) wm_v4s*)(&sm.v[kb][c0]));
          const wm_v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) wm_v4s*)(&sm.v[kb + 8][c0]));
          short8 a8;
          a8[0] = lo[0]; a8[1] = lo[1]; a8[2] = lo[2]; a8[3] = lo[3];
          a8[4] = hi[0]; a8[5] = hi[1]; a8[6] = hi[2]; a8[7] = hi[3];
          acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<bf16x8*>(&a8),
                                                            pf[t][s2], acc[dt], 0, 0, 0);
        }
    }
  }
  if (!valid) return;
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  bf16_t* orow = (bf16_t*)p.o + ((size_t)(q0 + qi) * p.H + head) * DV;
  const bf16_t* grow = p.gate ? (const bf16_t*)p.gate + (size_t)(q0 + qi) * p.gate_ld + (size_t)head * DV
                              : nullptr;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int g8 = 0; g8 < 4; ++g8) {
      const int d0 = 32 * dt + 8 * g8 + 4 * h;
      float o4[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) o4[i] = acc[dt][4 * g8 + i] * inv;
      if (grow) {
        const uint2 gw = *reinterpret_cast<const uint2*>(grow + d0);
        o4[0] *= sigmoid_fast(__uint_as_float(gw.x << 16));
        o4[1] *= sigmoid_fast(__uint_as_float(gw.x & 0xffff0000u));
        o4[2] *= sigmoid_fast(__uint_as_float(gw.y << 16));
        o4[3] *= sigmoid_fast(__uint_as_float(gw.y & 0xffff0000u));
      }
      uint2 w;
      w.x = pack_bf16x2(o4[0], o4[1]);
      w.y = pack_bf16x2(o4[2], o4[3]);
      *reinterpret_cast<uint2*>(orow + d0) = w;
    }
}

int window_attention_mfma(const WinAttnParams& p, int max_q, hipStream_t st) {
  if (max_q <= 0) return 0;
  const dim3 grid((max_q + WM_WAVES * 32 - 1) / (WM_WAVES * 32), p.H, p.B);
#define GO(A, C)                                                                              \
  if (p.D == A && p.Dv == C) {                                                                \
    hipLaunchKernelGGL((window_attn_mfma_kernel<A, C>), grid, dim3(WM_THREADS), 0, st, p);    \
    return (int)hipGetLastError();                                                            \
  }
  GO(64, 64) GO(128, 64) GO(64, 128) GO(128, 128)
#undef GO
  return (int)hipErrorInvalidValue;
}

// ------------------------------------------------------------------ launchers
extern "C" int loqa_qk_prep_append(const void* u, int dt, long ldu, int H, int G, int D, int Dv,
                                   int v_off, const void* cs, int max_pos, int dims, float eps,
                                   float coef, int every, const void* pos, void* kc, void* vc,
                                   int blk, int nblocks, const void* kvslots, void* q, int T,
                                   hipStream_t st) {
  if (T <= 0) return 0;
  if (D <= 0 || D > 512 || D % 2 || dims < 0 || dims > D || dims % 2 || every < 1 ||
      (dims > 0 && (!cs || max_pos <= 0)) || H <= 0 || G <= 0)
    return (int)hipErrorInvalidValue;
  const long rows = (long)blk * nblocks;
#define GO(TT)                                                                                  \
  hipLaunchKernelGGL(qk_prep_append_kernel<TT>, dim3(T), dim3(256), 0, st, (const TT*)u, ldu, H, \
                     G, D, Dv, v_off, (const float*)cs, max_pos, dims, eps, coef, every,        \
                     (const int*)pos, (TT*)kc, (TT*)vc, rows, (const int*)kvslots, (TT*)q)
  if (dt == 0) GO(bf16_t); else GO(float);
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_window_attention(const void* q, int dt, const void* kc, const void* vc, int blk,
                                     int nblocks, const void* cu_q, const void* ctx, const void* bt,
                                     int max_blocks, const void* pos, const void* gate, long gate_ld,
                                     float scale, float cap, int window, int keep_first, int B,
                                     int T, int H, int G, int D, int Dv, int max_q, int mfma,
                                     void* o, hipStream_t st) {
  if (T <= 0) return 0;
  if (B <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || D > 512 || Dv <= 0 || Dv > 512 || blk <= 0)
    return (int)hipErrorInvalidValue;
  WinAttnParams p;
  p.q = q; p.kc = kc; p.vc = vc; p.blk = blk; p.cache_rows = (long)blk * nblocks;
  p.cu_q = (const int*)cu_q; p.ctx = (const int*)ctx; p.bt = (const int*)bt;
  p.max_blocks = max_blocks; p.pos = (const int*)pos; p.gate = gate; p.gate_ld = gate_ld;
  p.scale = scale; p.cap = cap; p.window = window; p.keep_first = keep_first;
  p.B = B; p.T = T; p.H = H; p.G = G; p.D = D; p.Dv = Dv; p.o = o;
  // the matrix-core form reads the gate in 8-byte runs
  const bool gate_ok = !gate || (gate_ld % 4 == 0 && ((size_t)gate & 7) == 0);
  if (mfma && dt == 0 && (D == 64 || D == 128) && (Dv == 64 || Dv == 128) && gate_ok)
    return window_attention_mfma(p, max_q, st);
  const int rep = H / G;
  const int nv = Dv <= 128 ? 2 : 8;
  int R = rep >= 8 ? 8 : (rep >= 4 ? 4 : (rep >= 2 ? 2 : 1));
  if (nv == 8 && R > 4) R = 4;
  const dim3 grid(T, G, (rep + R - 1) / R);
  const size_t lds1 = (size_t)(R * D + WA_NW * R * 64) * 4;
  const size_t lds2 = (size_t)(2 * WA_NW * R + WA_NW * R * nv * 64) * 4;
  const size_t lds = lds1 > lds2 ? lds1 : lds2;
  if (lds > 64 * 1024) return (int)hipErrorInvalidValue;
#define GO(TT, RR, NN)                                                                         \
  hipLaunchKernelGGL((window_attn_keys_kernel<TT, RR, NN>), grid, dim3(64 * WA_NW), lds, st, p)
#define BY_R(TT, NN)                                                                           \
  do {                                                                                         \
    if (R == 8) GO(TT, 8, NN); else if (R == 4) GO(TT, 4, NN);                                 \
    else if (R == 2) GO(TT, 2, NN); else GO(TT, 1, NN);                                        \
  } while (0)
  if (dt == 0) { if (nv == 2) BY_R(bf16_t, 2); else BY_R(bf16_t, 8); }
  else { if (nv == 2) BY_R(float, 2); else BY_R(float, 8); }
#undef BY_R
#undef GO
  return (int)hipGetLastError();
}

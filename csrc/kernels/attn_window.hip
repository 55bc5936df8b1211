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
// positions, one per wave in turn (window index modulo the wave count; 16 waves
// when the launch has few workgroups, else 4). In a window, groups of D / 8
// lanes (D / 4 for f32) cover a key row in 16-byte runs, so one load brings
// whole rows; a lane multiplies its run with its part of q in registers, the
// group adds up with data-parallel moves, and one lane of the group keeps the
// key's score. An online softmax per head runs across the wave; the value rows
// are read in the same 16-byte runs, a lane sums its run over the rows of its
// group, and the groups are added once at the end. (Head sizes that are no
// power-of-two number of runs: a lane per key, a lane per output column.) The
// waves' partial (max, sum, accumulator) triples merge through LDS in wave
// order. Which windows a wave takes and the order of every sum depend only on
// the query's position and the wave count. When a step has few rows and long
// contexts the windows are also dealt out to several workgroups per row, whose
// partial triples a small combine launch merges.
//
// window_attn_mfma_kernel (bf16, D and Dv in {64, 128}; prompt portions): a
// workgroup per (64, 128 or 256 query rows of one sequence, query head); each
// wave owns 32 rows. The block-table entries of the key range go to LDS once.
// K and V tiles of 64 keys are gathered from the pages into LDS for all waves
// (the next tile's 16-byte chunks already in flight in registers);
// S^T = K Q^T and O^T += V^T P^T run on v_mfma_f32_32x32x16_bf16 with the query
// on the MFMA lane, so the online softmax is in-register. Tiles that lie wholly
// between the kept first tokens and the rows' windows are skipped, and a tile
// that every row of a wave sees whole takes a path without per-score tests.
#include "seqmix.h"

struct WinAttnParams {
  const void* q; const void* kc; const void* vc; int blk; long cache_rows;
  const int* cu_q; const int* ctx; const int* bt; int max_blocks; const int* pos;
  const void* gate; long gate_ld; float scale, cap; int window, keep_first;
  int B, T, H, G, D, Dv; void* o;
  int ns; float* part;               // key splits over workgroups and their partial results
  const float* sink;                 // [H] or null: exp(sink[h]) joins head h's softmax denominator
};

// K / V pages (and the block table) are read through pointers in the global
// address space: a load through a generic pointer counts against the LDS
// counter as well, so every wait for an LDS read would also wait for the cache
// rows in flight and the loads would run one after the other.
#define WA_GLOBAL __attribute__((address_space(1)))
typedef unsigned wa_u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct GAct;
template <> struct GAct<bf16_t> {
  static constexpr int N = 8;                     // elements of a 16-byte run
  static __device__ __forceinline__ float ld(const WA_GLOBAL bf16_t* p) { return bf2f(*p); }
  static __device__ __forceinline__ void ldv(const WA_GLOBAL bf16_t* p, float* f) {
    const wa_u32x4 v = *reinterpret_cast<const WA_GLOBAL wa_u32x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(v[i] << 16);
      f[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
  }
};
template <> struct GAct<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ float ld(const WA_GLOBAL float* p) { return *p; }
  static __device__ __forceinline__ void ldv(const WA_GLOBAL float* p, float* f) {
    const float4v v = *reinterpret_cast<const WA_GLOBAL float4v*>(p);
    f[0] = v[0]; f[1] = v[1]; f[2] = v[2]; f[3] = v[3];
  }
};

// Sum over groups of `gs` neighbouring lanes (a power of two): data-parallel
// moves inside rows of 16 lanes, shuffles above; every lane gets its group's sum.
template <int CTRL> __device__ __forceinline__ float wa_dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float wa_group_sum(float v, int gs) {
  if (gs >= 2) v += wa_dpp<0xB1>(v);              // lanes 1 0 3 2 of each four
  if (gs >= 4) v += wa_dpp<0x4E>(v);              // lanes 2 3 0 1 of each four
  if (gs >= 8) v += wa_dpp<0x141>(v);             // the other four of each eight (mirror)
  if (gs >= 16) v += wa_dpp<0x140>(v);            // the other eight of each sixteen (mirror)
  if (gs >= 32) v += __shfl_xor(v, 16, 64);
  if (gs >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

// The sequence of flat row t: the number of feed starts cu_q[1 .. B - 1] at or
// before t. Every lane tests one start, so a batch of up to 64 sequences costs
// one round trip instead of a chain of dependent loads (all lanes must be active).
__device__ __forceinline__ int wa_seq_of_row(const int* __restrict__ cu_q, int B, int t) {
  const int lane = threadIdx.x & 63;
  int b = 0;
  for (int base = 1; base < B; base += 64) {
    const int i = base + lane;
    const bool at_or_before = i < B && cu_q[i] <= t;
    b += __popcll(__ballot(at_or_before));
  }
  return b;
}

// ------------------------------------------------------------------ q / k rows
template <typename T>
__global__ __launch_bounds__(256) void qk_prep_append_kernel(
    const T* __restrict__ u, long ldu, int H, int G, int D, int Dv, int v_off,
    const float* __restrict__ cs, int max_pos, int dims, float eps, float coef, int every,
    const int* __restrict__ pos, T* __restrict__ kc, T* __restrict__ vc, long cache_rows,
    const int* __restrict__ kvslots, T* __restrict__ q, const float* __restrict__ qn,
    const float* __restrict__ kn) {
  __shared__ float wsum[2][4];
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int p = pos[t];
  const long slot = kvslots[t];
  const bool store = slot >= 0 && slot < cache_rows;
  const T* ur = u + (size_t)t * ldu;
  // the other norm: q and k RMS-normed over their whole projection, with
  // weights, before the rotation (then no per-head division)
  float invq = 1.f, invk = 1.f;
  if (qn) {
    float sq = 0.f, sk = 0.f;
    for (int c = threadIdx.x; c < (H + G) * D; c += blockDim.x) {
      const float v = Act<T>::ld(ur + c);
      if (c < H * D) sq += v * v; else sk += v * v;
    }
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    if (lane == 0) { wsum[0][wave] = sq; wsum[1][wave] = sk; }
    __syncthreads();
    invq = 1.f / sqrtf((wsum[0][0] + wsum[0][1] + wsum[0][2] + wsum[0][3]) / (float)(H * D) + eps);
    invk = 1.f / sqrtf((wsum[1][0] + wsum[1][1] + wsum[1][2] + wsum[1][3]) / (float)(G * D) + eps);
  }
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
        if (qn) {
          const float* wn = isq ? qn + (size_t)job * D + e : kn + (size_t)(job - H) * D + e;
          const float iv = isq ? invq : invk;
          a[i] *= iv * wn[0];
          b[i] *= iv * wn[1];
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
    float inv = qn ? 1.f : 1.f / sqrtf(ss / (float)D + eps);
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
template <typename T, int REP, int NV, int NW>
__global__ __launch_bounds__(64 * NW) void window_attn_keys_kernel(WinAttnParams p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x, g = blockIdx.y;
  if (t >= p.cu_q[p.B]) return;
  const int b = wa_seq_of_row(p.cu_q, p.B, t);
  const int D = p.D, Dv = p.Dv, rep = p.H / p.G;
  const int sp = blockIdx.z % p.ns;                // this block's share of the key windows
  const int r0 = (blockIdx.z / p.ns) * REP;        // first head of the group this block serves
  const int nr = min(REP, rep - r0);
  float* qs = lds;                                 // [REP][D]
  float* ws = qs + REP * D + wave * (REP + 1) * 64;   // per wave: weights [REP][64] ...
  int* rs = reinterpret_cast<int*>(ws + REP * 64);    // ... and the keys' cache rows [64]
  for (int i = threadIdx.x; i < REP * D; i += blockDim.x)
    qs[i] = i < nr * D ? Act<T>::ld((const T*)p.q + (size_t)t * p.H * D + (size_t)(g * rep + r0) * D + i)
                       : 0.f;
  __syncthreads();
  const int pq = p.pos[t];
  const int hi = min(pq, p.ctx[b] - 1);
  const int lo = p.window > 0 ? max(0, pq - p.window + 1) : 0;
  // windows of 64 keys: those that hold kept first tokens, then those from lo on
  const int w_lo = lo >> 6, w_hi = hi >> 6;
  const int n1 = p.window > 0 ? min((min(p.keep_first, lo) + 63) >> 6, w_lo) : 0;
  const int nwin = hi >= 0 ? n1 + (w_hi - w_lo + 1) : 0;
  const WA_GLOBAL int* bt = (const WA_GLOBAL int*)p.bt + (size_t)b * p.max_blocks;
  const WA_GLOBAL T* kc = (const WA_GLOBAL T*)p.kc;
  const WA_GLOBAL T* vc = (const WA_GLOBAL T*)p.vc;
  const size_t GD = (size_t)p.G * D, GDv = (size_t)p.G * Dv;
  constexpr int VN = GAct<T>::N;
  // value accumulators. NV > 0: a lane owns the output columns lane + 64 i.
  // NV == 0 (Dv / VN a power of two up to 64): LPR = Dv / VN lanes cover a value
  // row in 16-byte runs, so one load instruction brings 64 / LPR whole rows;
  // a lane sums its run over the rows of its lane group, and the groups are
  // added once at the end.
  constexpr bool ROWS = NV == 0;
  constexpr int NA = ROWS ? VN : NV;
  const int LPR = ROWS ? Dv / VN : 64;
  const int vrg = lane / LPR, vch = (lane % LPR) * VN;
  float m[REP], l[REP], acc[REP][NA];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
#pragma unroll
    for (int i = 0; i < NA; ++i) acc[r][i] = 0.f;
  }
  constexpr int KU = NW > 4 ? 4 : 8;                 // key / value row loads in flight per lane
  // key layout: LPK = D / VN lanes cover a key row in 16-byte runs when that is
  // a power of two up to 64 (else a lane per key, element by element); lane
  // group krg reads the rows krg, krg + 64 / LPK, ..., and the lane whose place
  // in the group equals the load's number owns that key from then on
  const int LPKc = D / VN;
  const bool krows = D % VN == 0 && LPKc <= 64 && (LPKc & (LPKc - 1)) == 0;
  const int LPK = krows ? LPKc : 64;
  const int krg = lane / LPK, kit = lane % LPK, kch = kit * VN;
  const int jl = krows ? kit * (64 / LPK) + krg : lane;   // the window's key this lane owns
  float qreg[REP][VN];
#pragma unroll
  for (int r = 0; r < REP; ++r)
#pragma unroll
    for (int i = 0; i < VN; ++i) qreg[r][i] = krows ? qs[r * D + kch + i] : 0.f;
  constexpr int VU = NV > 2 ? 4 : 8;                 // value rows in flight per lane (column form)
  for (int wk = sp * NW + wave; wk < nwin; wk += p.ns * NW) {
    const int k0 = (wk < n1 ? wk : w_lo + (wk - n1)) << 6;
    const int j = k0 + jl;
    const bool seen = j <= hi && (p.window <= 0 || pq - j < p.window || j < p.keep_first);
    // every lane names a valid cache row (past the end: the last key's), so the
    // loads below need no bounds tests; unseen keys weigh zero
    const int jc = min(j, hi);
    const long row = min(max((long)bt[jc / p.blk] * p.blk + jc % p.blk, 0L), p.cache_rows - 1);
    rs[jl] = (int)row;
    float s[REP];
#pragma unroll
    for (int r = 0; r < REP; ++r) s[r] = 0.f;
    if (krows) {
      // one load instruction brings 64 / LPK whole key rows; a lane multiplies its
      // 16-byte run with its part of q, the group adds up, the key's owner keeps it
      __builtin_amdgcn_wave_barrier();
      const int rpk = 64 / LPK;
      for (int i0 = 0; i0 < LPK; i0 += KU) {
        float f[KU][VN];
#pragma unroll
        for (int c = 0; c < KU; ++c) {
          const int kl = min((i0 + c) * rpk + krg, 63);
          GAct<T>::ldv(kc + (size_t)rs[kl] * GD + (size_t)g * D + kch, f[c]);
        }
#pragma unroll
        for (int c = 0; c < KU; ++c) {
#pragma unroll
          for (int r = 0; r < REP; ++r) {
            float d = 0.f;
#pragma unroll
            for (int i = 0; i < VN; ++i) d += qreg[r][i] * f[c][i];
            d = wa_group_sum(d, LPK);
            if (i0 + c == kit) s[r] = d;
          }
        }
      }
    } else if (seen) {
      const WA_GLOBAL T* kr = kc + (size_t)row * GD + (size_t)g * D;
      for (int e = 0; e < D; ++e) {
        const float f = GAct<T>::ld(kr + e);
#pragma unroll
        for (int r = 0; r < REP; ++r) s[r] += qs[r * D + e] * f;
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
      ws[r * 64 + jl] = e;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < REP; ++r)
#pragma unroll
      for (int i = 0; i < NA; ++i) acc[r][i] *= alpha[r];
    const int nk = min(64, hi - k0 + 1);
    if constexpr (ROWS) {
      const int rpi = 64 / LPR;                        // rows per load instruction
      for (int i0 = 0; i0 * rpi < nk; i0 += KU) {      // rows past nk weigh zero
        float v[KU][VN];
        int key[KU];
#pragma unroll
        for (int c = 0; c < KU; ++c) {
          key[c] = min((i0 + c) * rpi + vrg, 63);
          GAct<T>::ldv(vc + (size_t)rs[key[c]] * GDv + (size_t)g * Dv + vch, v[c]);
        }
#pragma unroll
        for (int c = 0; c < KU; ++c) {
          if ((i0 + c) * rpi >= 64) break;             // uniform: no rows left
#pragma unroll
          for (int r = 0; r < REP; ++r) {
            const float w = ws[r * 64 + key[c]];
#pragma unroll
            for (int i = 0; i < VN; ++i) acc[r][i] += w * v[c][i];
          }
        }
      }
    } else
    for (int kk = 0; kk < nk; kk += VU) {              // rows past nk weigh zero
      float v[VU][NA];
#pragma unroll
      for (int c = 0; c < VU; ++c) {
        const WA_GLOBAL T* vr = vc + (size_t)rs[kk + c] * GDv + (size_t)g * Dv;
#pragma unroll
        for (int i = 0; i < NA; ++i) {
          const int e = lane + 64 * i;
          v[c][i] = e < Dv ? GAct<T>::ld(vr + e) : 0.f;
        }
      }
#pragma unroll
      for (int c = 0; c < VU; ++c)
#pragma unroll
        for (int r = 0; r < REP; ++r) {
          const float w = ws[r * 64 + kk + c];
#pragma unroll
          for (int i = 0; i < NA; ++i) acc[r][i] += w * v[c][i];
        }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if constexpr (ROWS) {
    // add the lane groups: afterwards lanes 0 .. LPR - 1 hold the wave's sums
    for (int o = LPR; o < 64; o <<= 1)
#pragma unroll
      for (int r = 0; r < REP; ++r)
#pragma unroll
        for (int i = 0; i < NA; ++i) acc[r][i] += __shfl_xor(acc[r][i], o, 64);
  }
  // merge the waves' partials in wave order
  __syncthreads();                                   // qs / ws are free
  float* mm = lds;                                   // [NW][REP]
  float* ll = mm + NW * REP;                         // [NW][REP]
  float* aa = ll + NW * REP;                         // [NW][REP][Dv]
  if (lane == 0)
#pragma unroll
    for (int r = 0; r < REP; ++r) { mm[wave * REP + r] = m[r]; ll[wave * REP + r] = l[r]; }
#pragma unroll
  for (int r = 0; r < REP; ++r)
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int e = ROWS ? vch + i : lane + 64 * i;
      if (e < Dv && (!ROWS || lane < LPR)) aa[(size_t)(wave * REP + r) * Dv + e] = acc[r][i];
    }
  __syncthreads();
  for (int idx = threadIdx.x; idx < nr * Dv; idx += blockDim.x) {
    const int r = idx / Dv, e = idx - r * Dv;
    const int h = g * rep + r0 + r;
    const bool snk = p.sink && p.ns == 1;            // with key splits the combine launch adds it
    float M = snk ? p.sink[h] : -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, mm[w * REP + r]);
    float num = 0.f, den = snk ? expf(p.sink[h] - M) : 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = mm[w * REP + r];
      const float f = mw == -INFINITY ? 0.f : expf(mw - M);
      num += f * aa[(size_t)(w * REP + r) * Dv + e];
      den += f * ll[w * REP + r];
    }
    if (p.ns > 1) {                                  // the combine launch finishes the row
      float* pr = p.part + (((size_t)t * p.H + h) * p.ns + sp) * (Dv + 2);
      if (e == 0) { pr[0] = M; pr[1] = den; }
      pr[2 + e] = num;
      continue;
    }
    float out = den > 0.f ? num / den : 0.f;
    if (p.gate)
      out *= sigmoid_f(Act<T>::ld((const T*)p.gate + (size_t)t * p.gate_ld + (size_t)h * Dv + e));
    Act<T>::st((T*)p.o + (size_t)t * p.H * Dv + (size_t)h * Dv + e, out);
  }
}

// Merge of the key splits of a row: partials (max, sum, accumulator[Dv]) in
// split order, then the output gate.
template <typename T>
__global__ __launch_bounds__(128) void window_attn_combine_kernel(WinAttnParams p) {
  const int t = blockIdx.x, h = blockIdx.y, Dv = p.Dv;
  const float* pr = p.part + ((size_t)t * p.H + h) * p.ns * (Dv + 2);
  float M = p.sink ? p.sink[h] : -INFINITY;
  for (int s = 0; s < p.ns; ++s) M = fmaxf(M, pr[(size_t)s * (Dv + 2)]);
  for (int e = threadIdx.x; e < Dv; e += blockDim.x) {
    float num = 0.f, den = p.sink ? expf(p.sink[h] - M) : 0.f;
    for (int s = 0; s < p.ns; ++s) {
      const float* ps = pr + (size_t)s * (Dv + 2);
      const float f = ps[0] == -INFINITY ? 0.f : expf(ps[0] - M);
      num += f * ps[2 + e];
      den += f * ps[1];
    }
    float out = den > 0.f ? num / den : 0.f;
    if (p.gate)
      out *= sigmoid_f(Act<T>::ld((const T*)p.gate + (size_t)t * p.gate_ld + (size_t)h * Dv + e));
    Act<T>::st((T*)p.o + (size_t)t * p.H * Dv + (size_t)h * Dv + e, out);
  }
}

// ------------------------------------------------------------ prompt portions
#define WM_TILE 64
#define WM_MAXPG 2048                // block-table entries of a sequence kept in LDS

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

template <int DK, int DV, int WM_WAVES>
__global__ __launch_bounds__(64 * WM_WAVES) void window_attn_mfma_kernel(WinAttnParams p) {
  __shared__ __attribute__((aligned(16))) WinMfmaSmem<DK, DV> sm;
  __shared__ int pages[WM_MAXPG];
  constexpr int WM_THREADS = 64 * WM_WAVES;
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
  const WA_GLOBAL bf16_t* kbase = (const WA_GLOBAL bf16_t*)p.kc + (size_t)g * DK;
  const WA_GLOBAL bf16_t* vbase = (const WA_GLOBAL bf16_t*)p.vc + (size_t)g * DV;
  const WA_GLOBAL int* bt = (const WA_GLOBAL int*)p.bt + (size_t)b * p.max_blocks;
  // the pages of this workgroup's key range, looked up once
  const int npg = (kend + p.blk - 1) / p.blk;
  const bool pg_lds = npg <= WM_MAXPG;
  if (pg_lds) {
    for (int i = threadIdx.x; i < npg; i += WM_THREADS) pages[i] = bt[i];
    __syncthreads();
  }
  const float scale_log2 = p.scale * 1.4426950408889634f;
  const float cap_log2 = p.cap * 1.4426950408889634f, inv_cap = p.cap > 0.f ? p.scale / p.cap : 0.f;

  // K / V tiles go through registers: the next tile's 16-byte chunks are
  // requested before this tile's math and stored to LDS after it
  constexpr int NKC = WM_TILE * CHK / WM_THREADS, NVC = WM_TILE * CHV / WM_THREADS;
  wa_u32x4 pk[NKC], pv[NVC];
  // page size a power of two (the usual case): shifts instead of divisions
  const int pg_sh = (p.blk & (p.blk - 1)) == 0 ? __ffs(p.blk) - 1 : -1;
  auto page_row = [&](int j) -> size_t {
    const int pi = pg_sh >= 0 ? j >> pg_sh : j / p.blk;
    const long pg = pg_lds ? pages[pi] : bt[pi];
    return (size_t)min(max(pg * p.blk + (j - pi * p.blk), 0L), p.cache_rows - 1);
  };
  auto fetch = [&](int kt) {
#pragma unroll
    for (int j = 0; j < NKC; ++j) {
      const int c = threadIdx.x + WM_THREADS * j, kr = c / CHK, cc = (c - kr * CHK) * 8;
      pk[j] = kt + kr < kend
                  ? *reinterpret_cast<const WA_GLOBAL wa_u32x4*>(kbase + page_row(kt + kr) * kst + cc)
                  : wa_u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int j = 0; j < NVC; ++j) {
      const int c = threadIdx.x + WM_THREADS * j, kr = c / CHV, cc = (c - kr * CHV) * 8;
      pv[j] = kt + kr < kend
                  ? *reinterpret_cast<const WA_GLOBAL wa_u32x4*>(vbase + page_row(kt + kr) * vst + cc)
                  : wa_u32x4{0, 0, 0, 0};
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
      *reinterpret_cast<wa_u32x4*>(&sm.k[kr][cc]) = pk[j];
    }
#pragma unroll
    for (int j = 0; j < NVC; ++j) {
      const int c = threadIdx.x + WM_THREADS * j, kr = c / CHV, cc = (c - kr * CHV) * 8;
      *reinterpret_cast<wa_u32x4*>(&sm.v[kr][cc]) = pv[j];
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
      // a tile that every row of this wave sees whole needs no per-score tests
      const bool whole = kt + WM_TILE - 1 <= wpos_lo && kt + WM_TILE <= kend &&
                         (p.window <= 0 || wpos_hi - kt < p.window || kt + WM_TILE <= p.keep_first);
      if (whole) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            const float sv = p.cap > 0.f ? cap_log2 * tanh_fast(st[t][j] * inv_cap)
                                         : st[t][j] * scale_log2;
            st[t][j] = sv;
            mx = fmaxf(mx, sv);
          }
      } else {
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
      }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      // the hardware's exp2: the arguments are <= 0, and what falls below the
      // normal range may flush to zero
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      float ls = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float e = __builtin_amdgcn_exp2f(st[t][8 * s2 + j] - m_new);
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
  float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  if (p.sink) {
    // the running maximum and sum are in the base-2 domain
    const float sl = p.sink[head] * 1.44269504088896f;
    const float mx2 = fmaxf(m_run, sl);
    const float a = __builtin_amdgcn_exp2f(m_run - mx2);
    inv = a / (l_run * a + __builtin_amdgcn_exp2f(sl - mx2));
  }
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
  // the widest row block the longest feed fills: the tiles' staging (gather
  // through the page table, LDS stores, barriers) is paid once per block and
  // tile, and measured times fall with the block width even when the grid
  // shrinks below the number of compute units
  const int waves = max_q > 128 ? 8 : (max_q > 64 ? 4 : 2);
  const dim3 grid((max_q + waves * 32 - 1) / (waves * 32), p.H, p.B);
#define GO(A, C)                                                                              \
  if (p.D == A && p.Dv == C) {                                                                \
    if (waves == 8)                                                                           \
      hipLaunchKernelGGL((window_attn_mfma_kernel<A, C, 8>), grid, dim3(512), 0, st, p);      \
    else if (waves == 4)                                                                      \
      hipLaunchKernelGGL((window_attn_mfma_kernel<A, C, 4>), grid, dim3(256), 0, st, p);      \
    else                                                                                      \
      hipLaunchKernelGGL((window_attn_mfma_kernel<A, C, 2>), grid, dim3(128), 0, st, p);      \
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
                                   const void* qn, const void* kn, hipStream_t st) {
  if (T <= 0) return 0;
  if (D <= 0 || D > 512 || D % 2 || dims < 0 || dims > D || dims % 2 || every < 1 ||
      (dims > 0 && (!cs || max_pos <= 0)) || H <= 0 || G <= 0 || (!qn) != (!kn))
    return (int)hipErrorInvalidValue;
  const long rows = (long)blk * nblocks;
#define GO(TT)                                                                                  \
  hipLaunchKernelGGL(qk_prep_append_kernel<TT>, dim3(T), dim3(256), 0, st, (const TT*)u, ldu, H, \
                     G, D, Dv, v_off, (const float*)cs, max_pos, dims, eps, coef, every,        \
                     (const int*)pos, (TT*)kc, (TT*)vc, rows, (const int*)kvslots, (TT*)q,      \
                     (const float*)qn, (const float*)kn)
  if (dt == 0) GO(bf16_t); else GO(float);
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_window_attention(const void* q, int dt, const void* kc, const void* vc, int blk,
                                     int nblocks, const void* cu_q, const void* ctx, const void* bt,
                                     int max_blocks, const void* pos, const void* gate, long gate_ld,
                                     float scale, float cap, int window, int keep_first, int B,
                                     int T, int H, int G, int D, int Dv, int max_q, int mfma,
                                     void* o, int ns, void* part, const void* sink,
                                     hipStream_t st) {
  if (T <= 0) return 0;
  if (B <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || D > 512 || Dv <= 0 || Dv > 512 || blk <= 0)
    return (int)hipErrorInvalidValue;
  WinAttnParams p;
  p.q = q; p.kc = kc; p.vc = vc; p.blk = blk; p.cache_rows = (long)blk * nblocks;
  p.cu_q = (const int*)cu_q; p.ctx = (const int*)ctx; p.bt = (const int*)bt;
  p.max_blocks = max_blocks; p.pos = (const int*)pos; p.gate = gate; p.gate_ld = gate_ld;
  p.scale = scale; p.cap = cap; p.window = window; p.keep_first = keep_first;
  p.B = B; p.T = T; p.H = H; p.G = G; p.D = D; p.Dv = Dv; p.o = o;
  p.ns = 1; p.part = nullptr; p.sink = (const float*)sink;
  // the matrix-core form reads the gate in 8-byte runs
  const bool gate_ok = !gate || (gate_ld % 4 == 0 && ((size_t)gate & 7) == 0);
  if (mfma && dt == 0 && (D == 64 || D == 128) && (Dv == 64 || Dv == 128) && gate_ok)
    return window_attention_mfma(p, max_q, st);
  const int rep = H / G;
  // value layout: whole rows in 16-byte runs when Dv / (elements per run) is a
  // power of two up to 64, else a column per lane (2 or 8 columns)
  const int vn = dt == 0 ? 8 : 4, lpr = Dv / vn;
  const bool rows = Dv % vn == 0 && lpr <= 64 && (lpr & (lpr - 1)) == 0;
  const int nv = rows ? 0 : (Dv <= 128 ? 2 : 8);
  int R = rep >= 8 ? 8 : (rep >= 4 ? 4 : (rep >= 2 ? 2 : 1));
  if (nv == 8 && R > 4) R = 4;
  if (ns > 1 && part) { p.ns = ns; p.part = (float*)part; }
  const dim3 grid(T, G, (rep + R - 1) / R * p.ns);
  // few workgroups (decode steps): 16 waves share a row's keys, else 4
  auto lds_of = [&](int nw) {
    const size_t a = (size_t)(R * D + nw * (R + 1) * 64) * 4;
    const size_t b = (size_t)(2 * nw * R + nw * R * Dv) * 4;
    return a > b ? a : b;
  };
  int nw = rows && R <= 2 && p.ns == 1 && (long)grid.x * grid.y * grid.z < 256 ? 16 : 4;
  if (lds_of(nw) > 64 * 1024) nw = 4;
  const size_t lds = lds_of(nw);
  if (lds > 64 * 1024) return (int)hipErrorInvalidValue;
#define GO(TT, RR, NN, WW)                                                                     \
  hipLaunchKernelGGL((window_attn_keys_kernel<TT, RR, NN, WW>), grid, dim3(64 * WW), lds, st, p)
#define BY_R(TT, NN, WW)                                                                       \
  do {                                                                                         \
    if (R == 8) GO(TT, 8, NN, WW); else if (R == 4) GO(TT, 4, NN, WW);                         \
    else if (R == 2) GO(TT, 2, NN, WW); else GO(TT, 1, NN, WW);                                \
  } while (0)
#define BY_V(TT)                                                                               \
  do {                                                                                         \
    if (nv == 0 && nw == 16) BY_R(TT, 0, 16); else if (nv == 0) BY_R(TT, 0, 4);                \
    else if (nv == 2) BY_R(TT, 2, 4); else BY_R(TT, 8, 4);                                     \
  } while (0)
  if (dt == 0) BY_V(bf16_t); else BY_V(float);
#undef BY_V
#undef BY_R
#undef GO
  if (p.ns > 1) {
    if (dt == 0)
      hipLaunchKernelGGL(window_attn_combine_kernel<bf16_t>, dim3(T, H), dim3(128), 0, st, p);
    else
      hipLaunchKernelGGL(window_attn_combine_kernel<float>, dim3(T, H), dim3(128), 0, st, p);
  }
  return (int)hipGetLastError();
}

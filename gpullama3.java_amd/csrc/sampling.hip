// Token selection on the device: a row's softmax by many blocks, its choice by one.
//
// temperature == 0: the first index of the strictly greatest logit
//   (J/inference/sampler/Sampler.java:144-157).
// temperature > 0: p = softmax(logits / temperature) (Sampler.java:87-89), then
//   top_p outside (0,1): the first index whose running sum in index order exceeds
//     u, else the last index (J/inference/sampler/CategoricalSampler.java:31-42);
//   top_p inside (0,1): the tokens in descending order of probability (equal
//     ones by ascending index), cut after the first at which the running sum
//     exceeds top_p; u is scaled by the kept mass and the kept list is walked in
//     that order (J/inference/sampler/ToppSampler.java:116-155).
// The uniform number u in [0,1) comes from the caller, one per row.
//
// No sort: the kept set is {p > v} plus the first k of {p == v}, where v is the
// greatest threshold whose mass {p >= v} still exceeds top_p; v is found digit by
// digit over the float's bit pattern (four passes with histograms), and the walk to
// the drawn token is the same search with u * mass in place of top_p. Masses are
// summed as 64-bit integers (p * 2^62), so the order of a sum cannot move a comparison.
//
// At most 2^13 probabilities are 2^-13 or more. They are gathered while the row is normalised; when
// their mass alone exceeds top_p, the threshold and the drawn token lie among them and both searches
// walk that short list, in shared memory, instead of the row. A flat distribution, whose nucleus
// reaches further down, takes eight passes over the whole row.
#include "common.h"
#include "gl3_noalloc.h"
#include <mutex>

#define SB 1024
#define SW 16          // waves of a block
#define UN 16          // elements a thread asks for before it uses the first: a pass is bound by trips to memory
#define QSCALE 4611686018427387904.0   // 2^62: probabilities as 64-bit integers, sums exact and in any order
#define CAND_MAX 8192  // candidates kept in shared memory: the probabilities of at least CAND_CUT
#define CAND_CUT 0.0001220703125f      // 2^-13

// A probability (0 <= p <= 1) as an integer: floor(p * 2^62), exact for p >= 2^-38, truncated below;
// taken from the float's bits: mantissa shifted by its exponent.
__device__ __forceinline__ unsigned long long to_q(float p) {
  const uint32_t b = __float_as_uint(p);
  const int e = (int)(b >> 23) - 127;                    // p = 1.m * 2^e (e = -127: zero or denormal, taken as 0)
  if (e < -62) return 0ull;
  const unsigned long long m = (unsigned long long)((b & 0x7fffffu) | 0x800000u);   // 24 bits, value m * 2^(e-23)
  const int sh = 62 - 23 + e;                            // q = m * 2^sh
  return sh >= 0 ? m << sh : m >> -sh;
}

struct Found {
  uint32_t bits;               // the threshold value's bit pattern
  unsigned long long above;    // mass of the values greater than it
  unsigned long long each;     // the value as an integer
  int ties;                    // how many values equal it
};

// The greatest value v with mass{p >= v} > thr, found digit by digit over the float's bit pattern
// (8, 8, 8 and 7 bits): per digit one pass builds a histogram of mass and count over the values that
// share the digits found so far, in private per-wave tables (integer adds in shared memory), and
// wave 0 walks the 256 bins from the top. If no prefix of the values exceeds thr (thr is not below
// the total mass), the smallest value is returned.
template <typename Src>
__device__ Found radix_search(Src p, int V, unsigned long long thr,
                              unsigned long long (*h_mass)[256], int (*h_cnt)[256], unsigned long long* t_mass,
                              int* t_cnt, unsigned long long* res) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  uint32_t prefix = 0;
  unsigned long long above = 0;
  const int shifts[4] = {23, 15, 7, 0}, widths[4] = {8, 8, 8, 7};
  for (int level = 0; level < 4; ++level) {
    const int shift = shifts[level], width = widths[level];
    const uint32_t mask = (1u << width) - 1u;
    for (int i = tid; i < SW * 256; i += SB) { (&h_mass[0][0])[i] = 0; (&h_cnt[0][0])[i] = 0; }
    __syncthreads();
    for (int base = 0; base < V; base += UN * SB) {   // every lane stays in the loop: the wave votes below
      const int i0 = base + tid;
      float v[UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) v[u] = (i0 + u * SB < V) ? p[i0 + u * SB] : -1.f;
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const uint32_t b = __float_as_uint(v[u]);
        const bool in = v[u] >= 0.f && (b >> (shift + width)) == prefix;
        const int bin = (b >> shift) & mask;
        // a wave whose lanes all fall into one bin adds once
        const int first = __builtin_amdgcn_readfirstlane(in ? bin : -1);
        if (__all(in && bin == first)) {
          unsigned long long q = to_q(v[u]);
#pragma unroll
          for (int o = 32; o > 0; o >>= 1) q += __shfl_xor(q, o, 64);
          if (lane == 0) { atomicAdd(&h_mass[wave][bin], q); atomicAdd(&h_cnt[wave][bin], 64); }
        } else if (in) {
          atomicAdd(&h_mass[wave][bin], to_q(v[u]));
          atomicAdd(&h_cnt[wave][bin], 1);
        }
      }
    }
    __syncthreads();
    if (tid < 256) {
      unsigned long long m = 0;
      int c = 0;
      for (int w = 0; w < SW; ++w) { m += h_mass[w][tid]; c += h_cnt[w][tid]; }
      t_mass[tid] = m;
      t_cnt[tid] = c;
    }
    __syncthreads();
    if (wave == 0) {
      // lane l owns bins 255-4l .. 252-4l, walked downwards
      unsigned long long mine = 0;
      int cnt_mine = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) { mine += t_mass[255 - 4 * lane - k]; cnt_mine += t_cnt[255 - 4 * lane - k]; }
      unsigned long long incl = mine;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const unsigned long long y = __shfl_up(incl, o, 64);
        if (lane >= o) incl += y;
      }
      const bool crosses = above + incl > thr;
      const unsigned long long hit = __ballot(crosses);
      const unsigned long long some = __ballot(cnt_mine > 0);
      int who, bin = -1;
      unsigned long long cum = above + incl - mine;
      if (hit) {
        who = __ffsll((long long)hit) - 1;
        if (lane == who) {
          for (int k = 0; k < 4; ++k) {
            const int b = 255 - 4 * lane - k;
            if (cum + t_mass[b] > thr) { bin = b; break; }
            cum += t_mass[b];
          }
        }
      } else {
        who = 63 - __builtin_clzll(some);   // the lowest bins that hold anything
        if (lane == who) {
          for (int k = 3; k >= 0; --k) {
            const int b = 255 - 4 * lane - k;
            if (t_cnt[b] > 0) { bin = b; break; }
          }
          cum = above + incl;
          for (int k = 3; 255 - 4 * lane - k <= bin; --k) cum -= t_mass[255 - 4 * lane - k];
        }
      }
      if (lane == who) { res[0] = (unsigned long long)bin; res[1] = cum; }
    }
    __syncthreads();
    const int bin = (int)res[0];
    above = res[1];
    prefix = (prefix << width) | (uint32_t)bin;
    if (level == 3) {
      Found f;
      f.bits = prefix;
      f.above = above;
      f.ties = t_cnt[bin];
      f.each = f.ties ? t_mass[bin] / (unsigned long long)f.ties : 0;
      __syncthreads();
      return f;
    }
    __syncthreads();
  }
  return Found{};
}

// A row's softmax is made by many blocks, ST_SLICES slices a row, in three kernels (the maximum, the
// sum, the probabilities), before the row's one block picks the token: a single CU draws too few
// bytes a second, and has too little arithmetic, for a row of a hundred thousand logits. Rows with
// temperature 0 are left alone by the three.
#define ST_SLICES 64

// Scratch of a call, for every row: the probabilities; per slice the maximum, the sum of the
// exponentials and the mass as an integer; the candidates (probabilities of at least CAND_CUT) with
// their number and mass.
struct SampleWork {
  float* p;                        // [rows, V]
  double* slice_sum;               // [rows, ST_SLICES]
  unsigned long long* slice_mass;  // [rows, ST_SLICES]
  unsigned long long* cand_mass;   // [rows]
  float* slice_max;                // [rows, ST_SLICES]
  int* cand_count;                 // [rows]
  float* cand_p;                   // [rows, CAND_MAX]
  int* cand_i;                     // [rows, CAND_MAX]
};
#define SAMPLE_ROW_FLOATS (ST_SLICES * 5 + 4 + CAND_MAX * 2)   // beside the probabilities, 8-byte units kept whole

static SampleWork carve_sample_work(float* work, int n_rows, int V) {
  SampleWork w;
  w.p = work;
  w.slice_sum = (double*)(work + (((long)n_rows * V + 1) & ~1L));
  w.slice_mass = (unsigned long long*)(w.slice_sum + (long)n_rows * ST_SLICES);
  w.cand_mass = w.slice_mass + (long)n_rows * ST_SLICES;
  w.slice_max = (float*)(w.cand_mass + n_rows);
  w.cand_count = (int*)(w.slice_max + (long)n_rows * ST_SLICES);
  w.cand_p = (float*)(w.cand_count + n_rows);
  w.cand_i = (int*)(w.cand_p + (long)n_rows * CAND_MAX);
  return w;
}

__device__ __forceinline__ float row_max_of_slices(const float* slice_max, int row) {
  float m = slice_max[row * ST_SLICES + (threadIdx.x & (ST_SLICES - 1))];   // every wave holds all 64 slices
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  return m;
}

__global__ __launch_bounds__(256) void softmax_max_kernel(const float* __restrict__ logits, long ld,
                                                          const float* __restrict__ temperature, SampleWork w, int V) {
  __shared__ float fs[16];
  const int row = blockIdx.x, slice = blockIdx.y, tid = threadIdx.x;
  const float T = temperature[row];
  if (T == 0.f) return;
  if (slice == 0 && tid == 0) { w.cand_count[row] = 0; w.cand_mass[row] = 0ull; }   // for the third kernel
  const int per = (V + ST_SLICES - 1) / ST_SLICES;
  const int lo = min(V, slice * per), hi = min(V, lo + per);
  const float* lg = logits + (long)row * ld;
  float m = -INFINITY;
  for (int i = lo + tid; i < hi; i += 256) m = fmaxf(m, lg[i] / T);   // the division of the reference, per element
  m = block_max(m, fs);
  if (tid == 0) w.slice_max[row * ST_SLICES + slice] = m;
}

__global__ __launch_bounds__(256) void softmax_sum_kernel(const float* __restrict__ logits, long ld,
                                                          const float* __restrict__ temperature, SampleWork w, int V) {
  __shared__ double ds[16];
  const int row = blockIdx.x, slice = blockIdx.y, tid = threadIdx.x;
  const float T = temperature[row];
  if (T == 0.f) return;
  const float m = row_max_of_slices(w.slice_max, row);
  const int per = (V + ST_SLICES - 1) / ST_SLICES;
  const int lo = min(V, slice * per), hi = min(V, lo + per);
  const float* lg = logits + (long)row * ld;
  double z = 0.0;
  for (int i = lo + tid; i < hi; i += 256) z += (double)expf(lg[i] / T - m);
  z = block_sum_f64(z, ds);
  if (tid == 0) w.slice_sum[row * ST_SLICES + slice] = z;
}

// p = softmax(logits / T) into the scratch, each slice's mass as an integer, and the candidates.
__global__ __launch_bounds__(256) void softmax_prob_kernel(const float* __restrict__ logits, long ld,
                                                           const float* __restrict__ temperature,
                                                           const float* __restrict__ top_p, SampleWork w, int V) {
  __shared__ unsigned long long qs[2][4];
  __shared__ float bc_p[8 * 256];
  __shared__ int bc_i[8 * 256];
  __shared__ int bc_n, bc_base;
  const int row = blockIdx.x, slice = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
  const float T = temperature[row];
  if (T == 0.f) return;
  const float m = row_max_of_slices(w.slice_max, row);
  double z = 0.0;
  for (int k = 0; k < ST_SLICES; ++k) z += w.slice_sum[row * ST_SLICES + k];   // one order for every thread
  const float zf = (float)z;
  const float tp = top_p[row];
  const bool nucleus = tp > 0.f && tp < 1.f;
  const int per = (V + ST_SLICES - 1) / ST_SLICES;
  const int lo = min(V, slice * per), hi = min(V, lo + per);
  const float* lg = logits + (long)row * ld;
  float* p = w.p + (long)row * V;
  unsigned long long mass = 0, cmass = 0;
  for (int base = lo; base < hi; base += 8 * 256) {
    if (nucleus) {
      if (tid == 0) bc_n = 0;
      __syncthreads();
    }
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) { const int i = base + u * 256 + tid; v[u] = i < hi ? lg[i] : 0.f; }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = base + u * 256 + tid;
      if (i < hi) {
        const float pv = expf(v[u] / T - m) / zf;
        const unsigned long long q = to_q(pv);
        p[i] = pv;
        mass += q;
        if (nucleus && pv >= CAND_CUT) {
          const int slot = atomicAdd(&bc_n, 1);   // at most 8 * 256 of them
          bc_p[slot] = pv;
          bc_i[slot] = i;
          cmass += q;
        }
      }
    }
    if (nucleus) {
      // the block's candidates of this stretch go to the row's list with one addition to its counter
      __syncthreads();
      const int n = bc_n;
      if (tid == 0 && n > 0) bc_base = atomicAdd(&w.cand_count[row], n);
      __syncthreads();
      for (int k = tid; k < n; k += 256) {
        const int slot = bc_base + k;
        if (slot < CAND_MAX) {
          w.cand_p[(long)row * CAND_MAX + slot] = bc_p[k];
          w.cand_i[(long)row * CAND_MAX + slot] = bc_i[k];
        }
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { mass += __shfl_xor(mass, o, 64); cmass += __shfl_xor(cmass, o, 64); }
  if (lane == 0) { qs[0][tid >> 6] = mass; qs[1][tid >> 6] = cmass; }
  __syncthreads();
  if (tid == 0) {
    w.slice_mass[row * ST_SLICES + slice] = qs[0][0] + qs[0][1] + qs[0][2] + qs[0][3];
    const unsigned long long c = qs[1][0] + qs[1][1] + qs[1][2] + qs[1][3];
    if (c) atomicAdd(&w.cand_mass[row], c);   // integers: the order does not matter
  }
}

// The choice, one block a row.
__global__ __launch_bounds__(SB) void sample_kernel(const float* __restrict__ logits, long ld, SampleWork w,
                                                    const float* __restrict__ temperature,
                                                    const float* __restrict__ top_p, const float* __restrict__ uniform,
                                                    int* __restrict__ out, int V, const int* __restrict__ step,
                                                    int uniform_stride) {
  __shared__ float fs[16];
  __shared__ int is[16];
  __shared__ unsigned long long h_mass[SW][256];
  __shared__ int h_cnt[SW][256];
  __shared__ unsigned long long t_mass[256];
  __shared__ int t_cnt[256];
  __shared__ unsigned long long res[2];
  __shared__ unsigned long long w_tot[SW];
  __shared__ int winner;
  __shared__ float cand_p[CAND_MAX];
  __shared__ int cand_i[CAND_MAX];
  __shared__ unsigned long long t_q[SB];
  const int row = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const float* lg = logits + (long)row * ld;
  const float T = temperature[row];

  if (T == 0.f) {
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = tid; i < V; i += SB) {
      const float v = lg[i];
      if (v > best) { best = v; idx = i; }
    }
    // reduce (best, idx): greater value wins, equal values: lower index
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(idx, o, 64);
      if (ob > best || (ob == best && oi < idx)) { best = ob; idx = oi; }
    }
    if ((tid & 63) == 0) { fs[tid >> 6] = best; is[tid >> 6] = idx; }
    __syncthreads();
    if (tid == 0) {
      for (int w2 = 1; w2 < SB / 64; ++w2)
        if (fs[w2] > best || (fs[w2] == best && is[w2] < idx)) { best = fs[w2]; idx = is[w2]; }
      out[row] = idx == 0x7fffffff ? 0 : idx;   // all -inf or NaN: index 0, as the reference's loop leaves it
    }
    return;
  }

  const float* p = w.p + (long)row * V;
  const float tp = top_p[row];
  // in a run of steps replayed from a graph the step's number is read from memory
  const double u = (double)uniform[(step ? (long)step[0] * uniform_stride : 0) + row];
  if (tid == 0) winner = -1;
  __syncthreads();

  if (tp <= 0.f || tp >= 1.f) {
    // the first index whose running sum in index order exceeds u: first the slice, by the slices' masses
    const unsigned long long uq = (unsigned long long)(u * QSCALE);   // u = k / 2^24: exact
    const unsigned long long sm = w.slice_mass[row * ST_SLICES + lane];
    unsigned long long sincl = sm;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const unsigned long long y = __shfl_up(sincl, o, 64);
      if (lane >= o) sincl += y;
    }
    const unsigned long long shit = __ballot(uq < sincl);
    if (!shit) {                      // u lies beyond the whole mass: the last index
      if (tid == 0) out[row] = V - 1;
      return;
    }
    const int slice = __ffsll((long long)shit) - 1;
    const unsigned long long before_slice = __shfl(sincl - sm, slice, 64);
    const int sper = (V + ST_SLICES - 1) / ST_SLICES;
    const int r_lo = min(V, slice * sper), r_hi = min(V, r_lo + sper);
    // every wave owns a contiguous part of the slice, a multiple of 64 long
    const int per = ((r_hi - r_lo + SW - 1) / SW + 63) / 64 * 64;
    const int lo = min(r_hi, r_lo + wave * per), hi = min(r_hi, lo + per);
    unsigned long long mine = 0;
    for (int i0 = lo + lane; i0 < hi; i0 += 8 * 64) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = (i0 + 64 * k < hi) ? p[i0 + 64 * k] : 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) mine += to_q(v[k]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o, 64);
    if (lane == 0) w_tot[wave] = mine;
    __syncthreads();
    unsigned long long before = before_slice;
    for (int w2 = 0; w2 < wave; ++w2) before += w_tot[w2];
    if (before <= uq && uq < before + w_tot[wave]) {       // the crossing lies in this wave's part
      for (int base = lo; base < hi; base += 64) {
        const int i = base + lane;
        const unsigned long long q = i < hi ? to_q(p[i]) : 0;
        unsigned long long incl = q;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
          const unsigned long long y = __shfl_up(incl, o, 64);
          if (lane >= o) incl += y;
        }
        const unsigned long long hit = __ballot(uq < before + incl);
        if (hit) {
          if (lane == 0) winner = base + __ffsll((long long)hit) - 1;
          break;
        }
        before += __shfl(incl, 63, 64);
      }
    }
    __syncthreads();
    if (tid == 0) out[row] = winner >= 0 ? winner : V - 1;
    return;
  }

  // nucleus: the threshold value, the mass above it, and how many of the equal ones are kept
  const unsigned long long tq = (unsigned long long)((double)tp * QSCALE);
  const int n_cand = w.cand_count[row];
  if (n_cand <= CAND_MAX && w.cand_mass[row] > tq) {
    // the candidates alone exceed top_p: every probability from the threshold upwards is among them
    const int n = n_cand;
    for (int a = tid; a < n; a += SB) {
      cand_p[a] = w.cand_p[(long)row * CAND_MAX + a];
      cand_i[a] = w.cand_i[(long)row * CAND_MAX + a];
    }
    __syncthreads();
    if (n <= SB) {
      // few candidates, one a thread: the mass that stands before each in the kept order (descending
      // probability, equal ones by ascending index) is summed directly. A candidate is kept if the
      // mass before it does not exceed top_p; the drawn one is that whose stretch holds u * kept mass.
      float pa = 0.f;
      int ia = 0;
      unsigned long long qa = 0;
      if (tid < n) { pa = cand_p[tid]; ia = cand_i[tid]; qa = to_q(pa); }
      if (tid < n) t_q[tid] = qa;
      if (tid == 0) res[0] = w.cand_mass[row];
      __syncthreads();
      unsigned long long excl = 0;
      if (tid < n)
        for (int b = 0; b < n; ++b) {
          const float pb = cand_p[b];
          excl += (pb > pa || (pb == pa && cand_i[b] < ia)) ? t_q[b] : 0ull;
        }
      if (tid < n && excl <= tq && tq < excl + qa) res[0] = excl + qa;   // the last kept one: the kept mass
      __syncthreads();
      const unsigned long long target = (unsigned long long)(u * (double)res[0]);
      if (tid < n && excl <= target && target < excl + qa) winner = ia;
      __syncthreads();
      if (tid == 0) out[row] = winner >= 0 ? winner : V - 1;
      return;
    }
    const Found f1 = radix_search(cand_p, n, tq, h_mass, h_cnt, t_mass, t_cnt, res);
    long k1 = 1;
    if (f1.each > 0 && tq >= f1.above) k1 = (long)((tq - f1.above) / f1.each) + 1;
    if (k1 > f1.ties) k1 = f1.ties;
    if (k1 < 1) k1 = 1;
    const unsigned long long mass = f1.above + (unsigned long long)k1 * f1.each;
    const unsigned long long target = (unsigned long long)(u * (double)mass);
    const Found f2 = radix_search(cand_p, n, target, h_mass, h_cnt, t_mass, t_cnt, res);
    long j = (f2.each > 0 && target >= f2.above) ? (long)((target - f2.above) / f2.each) : 0;
    const long limit = (f2.bits == f1.bits) ? k1 : (long)f2.ties;
    if (j > limit - 1) j = limit - 1;
    if (j < 0) j = 0;
    const float want = __uint_as_float(f2.bits);
    // the candidate with this probability that has exactly j equal ones of smaller index before it
    for (int a = tid; a < n; a += SB) {
      if (cand_p[a] != want) continue;
      const int ia = cand_i[a];
      long rank = 0;
      for (int b = 0; b < n; ++b) rank += (cand_p[b] == want && cand_i[b] < ia) ? 1 : 0;
      if (rank == j) winner = ia;
    }
    __syncthreads();
    if (tid == 0) out[row] = winner >= 0 ? winner : V - 1;
    return;
  }
  const Found f1 = radix_search(p, V, tq, h_mass, h_cnt, t_mass, t_cnt, res);
  long k1 = 1;
  if (f1.each > 0 && tq >= f1.above) k1 = (long)((tq - f1.above) / f1.each) + 1;   // smallest k with above + k*each > tq
  if (k1 > f1.ties) k1 = f1.ties;
  if (k1 < 1) k1 = 1;
  const unsigned long long mass = f1.above + (unsigned long long)k1 * f1.each;
  // the drawn token: first in the kept order whose running sum exceeds u * mass
  const unsigned long long target = (unsigned long long)(u * (double)mass);
  const Found f2 = radix_search(p, V, target, h_mass, h_cnt, t_mass, t_cnt, res);
  long j = (f2.each > 0 && target >= f2.above) ? (long)((target - f2.above) / f2.each) : 0;
  const long limit = (f2.bits == f1.bits) ? k1 : (long)f2.ties;
  if (j > limit - 1) j = limit - 1;
  if (j < 0) j = 0;
  const float want_value = __uint_as_float(f2.bits);   // the drawn token is the `want_index`-th (from 0) with this
  const long want_index = j;                           // probability, in ascending order of index

  // every wave owns a contiguous range of the row, a multiple of 64 long
  const int per = ((V + SW - 1) / SW + 63) / 64 * 64;
  const int lo = min(V, wave * per), hi = min(V, lo + per);
  int mine = 0;
  for (int i0 = lo + lane; i0 < hi; i0 += 8 * 64) {
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = (i0 + 64 * k < hi) ? p[i0 + 64 * k] : -1.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) mine += (v[k] == want_value) ? 1 : 0;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o, 64);
  if (lane == 0) w_tot[wave] = (unsigned long long)mine;
  __syncthreads();
  long before = 0;
  for (int w2 = 0; w2 < wave; ++w2) before += (long)w_tot[w2];
  if (before <= want_index && want_index < before + (long)w_tot[wave]) {
    for (int base = lo; base < hi; base += 64) {
      const int i = base + lane;
      const unsigned long long hit = __ballot(i < hi && p[i] == want_value);
      const int n = __popcll(hit);
      if (want_index < before + n) {
        if (lane == 0) {
          unsigned long long h = hit;
          for (long skip = want_index - before; skip > 0; --skip) h &= h - 1;   // drop the lowest set bits
          winner = base + __ffsll((long long)h) - 1;
        }
        break;
      }
      before += n;
    }
  }
  __syncthreads();
  if (tid == 0) out[row] = winner >= 0 ? winner : V - 1;
}

// Greedy rows only, in two stages so that a row is read by many blocks at once: each block finds the
// first greatest logit of its slice, a second kernel the first greatest of the slices' results.
#define ARG_SLICES 64

__global__ __launch_bounds__(256) void argmax_slice_kernel(const float* __restrict__ logits, long ld,
                                                           float* __restrict__ part_val, int* __restrict__ part_idx,
                                                           int V) {
  __shared__ float fs[4];
  __shared__ int is[4];
  const int row = blockIdx.x, slice = blockIdx.y, tid = threadIdx.x;
  const int per = (V + ARG_SLICES - 1) / ARG_SLICES;
  const int lo = slice * per, hi = min(V, lo + per);
  const float* lg = logits + (long)row * ld;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = lo + tid; i < hi; i += 256) {
    const float v = lg[i];
    if (v > best) { best = v; idx = i; }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(idx, o, 64);
    if (ob > best || (ob == best && oi < idx)) { best = ob; idx = oi; }
  }
  if ((tid & 63) == 0) { fs[tid >> 6] = best; is[tid >> 6] = idx; }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 4; ++w)
      if (fs[w] > best || (fs[w] == best && is[w] < idx)) { best = fs[w]; idx = is[w]; }
    part_val[row * ARG_SLICES + slice] = best;
    part_idx[row * ARG_SLICES + slice] = idx;
  }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ part_val,
                                                          const int* __restrict__ part_idx, int* __restrict__ out) {
  const int row = blockIdx.x, lane = threadIdx.x;
  float best = part_val[row * ARG_SLICES + lane];
  int idx = part_idx[row * ARG_SLICES + lane];
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(idx, o, 64);
    if (ob > best || (ob == best && oi < idx)) { best = ob; idx = oi; }
  }
  if (lane == 0) out[row] = idx == 0x7fffffff ? 0 : idx;
}

// Every row greedy (J/inference/sampler/Sampler.java:144-157). work: at least 2 * n_rows * 64 floats.
extern "C" int gl3_argmax(const float* logits, long ld, float* work, int* out, int n_rows, int V, hipStream_t stream) {
  if (n_rows == 0) return 0;
  GL3_REQUIRE(logits && work && out && n_rows > 0 && V > 0 && ld >= V, "gl3_argmax: bad arguments");
  GL3_REQUIRE(n_rows <= 65535, "gl3_argmax: too many rows");
  float* pv = work;
  int* pi = (int*)(work + (long)n_rows * ARG_SLICES);
  argmax_slice_kernel<<<dim3(n_rows, ARG_SLICES), dim3(256), 0, stream>>>(logits, ld, pv, pi, V);
  GL3_LAUNCH_CHECK();
  argmax_final_kernel<<<dim3(n_rows), dim3(64), 0, stream>>>(pv, pi, out);
  GL3_LAUNCH_CHECK();
  return 0;
}

// The greedy pick of a decode step inside a run, and what follows it between two steps of the run (as
// gl3_decode_advance does): each row's winner is the sequence's next token, goes into row step[0] of `history`, the
// sequence moves on by one position, and the step counter goes up. One block does the second stage for all rows
// (a wave a row, in turn), so the counter is read by everyone before it changes: one launch instead of two.
__global__ __launch_bounds__(1024) void argmax_final_advance_kernel(const float* __restrict__ part_val,
                                                                    const int* __restrict__ part_idx, int* __restrict__ out,
                                                                    int n_rows, int* __restrict__ token_ids,
                                                                    int* __restrict__ positions, int* __restrict__ kv_before,
                                                                    int* __restrict__ history, int history_stride,
                                                                    int* __restrict__ step) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int s = step[0];
  __syncthreads();
  for (int row = wave; row < n_rows; row += 16) {
    float best = part_val[row * ARG_SLICES + lane];
    int idx = part_idx[row * ARG_SLICES + lane];
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(idx, o, 64);
      if (ob > best || (ob == best && oi < idx)) { best = ob; idx = oi; }
    }
    if (lane == 0) {
      const int t = idx == 0x7fffffff ? 0 : idx;
      out[row] = t;
      token_ids[row] = t;
      history[(long)s * history_stride + row] = t;
      positions[row] += 1;
      kv_before[row] += 1;
    }
  }
  if (threadIdx.x == 0) step[0] = s + 1;
}

extern "C" int gl3_argmax_advance(const float* logits, long ld, float* work, int* out, int n_rows, int V, int* token_ids,
                                  int* positions, int* kv_before, int* history, int history_stride, int* step,
                                  hipStream_t stream) {
  if (n_rows == 0) return 0;
  GL3_REQUIRE(logits && work && out && n_rows > 0 && V > 0 && ld >= V, "gl3_argmax_advance: bad arguments");
  GL3_REQUIRE(token_ids && positions && kv_before && history && step && history_stride >= n_rows && n_rows <= 1024,
              "gl3_argmax_advance: rows=%d stride=%d", n_rows, history_stride);
  float* pv = work;
  int* pi = (int*)(work + (long)n_rows * ARG_SLICES);
  argmax_slice_kernel<<<dim3(n_rows, ARG_SLICES), dim3(256), 0, stream>>>(logits, ld, pv, pi, V);
  GL3_LAUNCH_CHECK();
  argmax_final_advance_kernel<<<dim3(1), dim3(1024), 0, stream>>>(pv, pi, out, n_rows, token_ids, positions, kv_before,
                                                                  history, history_stride, step);
  GL3_LAUNCH_CHECK();
  return 0;
}

// The same without a workspace from the caller (see gl3_noalloc.h): the slices' partial results live
// in a device array of this library. In host code `scratch` is only a handle for the runtime, not a
// device address; the address on each GPU is asked for once, with that GPU current, and kept.
static __device__ __align__(256) float scratch[GL3_ARGMAX_STATIC_ROWS * 2 * ARG_SLICES];
#define GL3_MAX_DEVICES 64
static float* g_scratch_ptr[GL3_MAX_DEVICES];
static std::mutex g_scratch_mutex;

extern "C" int gl3_argmax_static(const float* logits, long ld, int* out, int n_rows, int V, hipStream_t stream) {
  if (n_rows == 0) return 0;
  GL3_REQUIRE(logits && out && n_rows > 0 && V > 0 && ld >= V, "gl3_argmax_static: bad arguments");
  GL3_REQUIRE(n_rows <= GL3_ARGMAX_STATIC_ROWS, "gl3_argmax_static: %d rows exceed the %d that the library's array holds",
              n_rows, GL3_ARGMAX_STATIC_ROWS);
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  GL3_REQUIRE(e == hipSuccess && dev >= 0 && dev < GL3_MAX_DEVICES, "gl3_argmax_static: no current device (%s)",
              hipGetErrorString(e));
  float* work;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      GL3_REQUIRE(e == hipSuccess && p != nullptr, "gl3_argmax_static: the array's address on device %d: %s", dev,
                  hipGetErrorString(e));
      g_scratch_ptr[dev] = (float*)p;
    }
    work = g_scratch_ptr[dev];
  }
  float* pv = work;
  int* pi = (int*)(work + (long)GL3_ARGMAX_STATIC_ROWS * ARG_SLICES);
  argmax_slice_kernel<<<dim3(n_rows, ARG_SLICES), dim3(256), 0, stream>>>(logits, ld, pv, pi, V);
  GL3_LAUNCH_CHECK();
  argmax_final_kernel<<<dim3(n_rows), dim3(64), 0, stream>>>(pv, pi, out);
  GL3_LAUNCH_CHECK();
  return 0;
}

// Floats of scratch that gl3_sample needs: the rows' probabilities and, per row, what the kernels
// hand to each other.
extern "C" long gl3_sample_work_floats(int n_rows, int V) {
  return (((long)n_rows * V + 1) & ~1L) + (long)n_rows * SAMPLE_ROW_FLOATS;
}

// work: gl3_sample_work_floats(n_rows, V) floats of scratch, 8-byte aligned.
// step (may be null): a counter in device memory; row r then takes uniform[step[0] * uniform_stride + r].
extern "C" int gl3_sample(const float* logits, long ld, float* work, const float* temperature, const float* top_p,
                          const float* uniform, int* out, int n_rows, int V, const int* step, int uniform_stride,
                          hipStream_t stream) {
  if (n_rows == 0) return 0;
  GL3_REQUIRE(logits && work && temperature && top_p && uniform && out, "gl3_sample: null argument");
  GL3_REQUIRE(n_rows > 0 && n_rows <= 65535 && V > 0 && ld >= V, "gl3_sample: bad sizes (rows=%d V=%d ld=%ld)", n_rows, V,
              ld);
  GL3_REQUIRE((uintptr_t)work % 8 == 0, "gl3_sample: the scratch must be 8-byte aligned");
  const SampleWork w = carve_sample_work(work, n_rows, V);
  const dim3 slices(n_rows, ST_SLICES);
  softmax_max_kernel<<<slices, dim3(256), 0, stream>>>(logits, ld, temperature, w, V);
  GL3_LAUNCH_CHECK();
  softmax_sum_kernel<<<slices, dim3(256), 0, stream>>>(logits, ld, temperature, w, V);
  GL3_LAUNCH_CHECK();
  softmax_prob_kernel<<<slices, dim3(256), 0, stream>>>(logits, ld, temperature, top_p, w, V);
  GL3_LAUNCH_CHECK();
  sample_kernel<<<dim3(n_rows), dim3(SB), 0, stream>>>(logits, ld, w, temperature, top_p, uniform, out, V, step,
                                                       uniform_stride);
  GL3_LAUNCH_CHECK();
  return 0;
}

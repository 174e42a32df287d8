// Token selection on the device: one block per row of logits.
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
// At most 2^13 probabilities are 2^-13 or more. They are gathered in shared memory while the row
// is normalised; when their mass alone exceeds top_p, the threshold and the drawn token lie among
// them and both searches walk that short list instead of the row: three passes over the row in
// place of twelve. A flat distribution, whose nucleus reaches further down, takes the passes over
// the whole row.
#include "common.h"

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

__global__ __launch_bounds__(SB) void sample_kernel(const float* __restrict__ logits, long ld, float* __restrict__ work,
                                                    const float* __restrict__ temperature,
                                                    const float* __restrict__ top_p, const float* __restrict__ uniform,
                                                    int* __restrict__ out, int V, const int* __restrict__ step,
                                                    int uniform_stride) {
  __shared__ float fs[16];
  __shared__ int is[16];
  __shared__ double ds[16];
  __shared__ unsigned long long h_mass[SW][256];
  __shared__ int h_cnt[SW][256];
  __shared__ unsigned long long t_mass[256];
  __shared__ int t_cnt[256];
  __shared__ unsigned long long res[2];
  __shared__ unsigned long long w_tot[SW];
  __shared__ int winner;
  __shared__ float cand_p[CAND_MAX];
  __shared__ int cand_i[CAND_MAX];
  __shared__ int n_cand;
  __shared__ unsigned long long cand_mass;
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
      for (int w = 1; w < SB / 64; ++w)
        if (fs[w] > best || (fs[w] == best && is[w] < idx)) { best = fs[w]; idx = is[w]; }
      out[row] = idx == 0x7fffffff ? 0 : idx;   // all -inf or NaN: index 0, as the reference's loop leaves it
    }
    return;
  }

  // p = softmax(logits / T), kept in `work`
  float* p = work + (long)row * V;
  float m = -INFINITY;
  for (int i0 = tid; i0 < V; i0 += UN * SB) {
    float v[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) v[u] = (i0 + u * SB < V) ? lg[i0 + u * SB] : -INFINITY;
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const float sc = v[u] / T;                          // the division of the reference, once per element
      if (i0 + u * SB < V) p[i0 + u * SB] = sc;
      m = fmaxf(m, sc);
    }
  }
  m = block_max(m, fs);
  double z = 0.0;
  for (int i0 = tid; i0 < V; i0 += UN * SB) {
    float v[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) v[u] = (i0 + u * SB < V) ? p[i0 + u * SB] : 0.f;
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int i = i0 + u * SB;
      if (i < V) {
        const float e = expf(v[u] - m);
        p[i] = e;
        z += (double)e;
      }
    }
  }
  const float zf = (float)block_sum_f64(z, ds);
  const float tp = top_p[row];
  const bool nucleus = tp > 0.f && tp < 1.f;
  if (tid == 0) { n_cand = 0; cand_mass = 0ull; }
  __syncthreads();
  unsigned long long my_mass = 0;
  for (int i0 = tid; i0 < V; i0 += UN * SB) {
    float v[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) v[u] = (i0 + u * SB < V) ? p[i0 + u * SB] : 0.f;
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int i = i0 + u * SB;
      if (i < V) {
        const float pv = v[u] / zf;
        p[i] = pv;
        if (nucleus && pv >= CAND_CUT) {
          const int slot = atomicAdd(&n_cand, 1);
          if (slot < CAND_MAX) { cand_p[slot] = pv; cand_i[slot] = i; }
          my_mass += to_q(pv);
        }
      }
    }
  }
  if (nucleus && my_mass) atomicAdd(&cand_mass, my_mass);   // integers: the order does not matter
  __syncthreads();

  // in a run of steps replayed from a graph the step's number is read from memory
  const double u = (double)uniform[(step ? (long)step[0] * uniform_stride : 0) + row];
  // every wave owns a contiguous range of the row, a multiple of 64 long
  const int per = ((V + SW - 1) / SW + 63) / 64 * 64;
  const int lo = min(V, wave * per), hi = min(V, lo + per);
  if (tid == 0) winner = -1;

  float want_value = 0.f;             // top-p: the drawn token is the `want_index`-th (from 0) with this probability
  long want_index = 0;
  if (tp <= 0.f || tp >= 1.f) {
    // the first index whose running sum in index order exceeds u
    const unsigned long long uq = (unsigned long long)(u * QSCALE);   // u = k / 2^24: exact
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
    unsigned long long before = 0;
    for (int w = 0; w < wave; ++w) before += w_tot[w];
    if (before <= uq && uq < before + w_tot[wave]) {       // the crossing lies in this wave's range
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
  if (n_cand <= CAND_MAX && cand_mass > tq) {
    // the candidates alone exceed top_p: every probability from the threshold upwards is among them
    const int n = n_cand;
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
  want_value = __uint_as_float(f2.bits);
  want_index = j;

  // the want_index-th index, in ascending order, whose probability is want_value
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
  for (int w = 0; w < wave; ++w) before += (long)w_tot[w];
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

// work: [n_rows, V] floats of scratch (probabilities); unused for greedy rows.
// step (may be null): a counter in device memory; row r then takes uniform[step[0] * uniform_stride + r].
extern "C" int gl3_sample(const float* logits, long ld, float* work, const float* temperature, const float* top_p,
                          const float* uniform, int* out, int n_rows, int V, const int* step, int uniform_stride,
                          hipStream_t stream) {
  if (n_rows == 0) return 0;
  GL3_REQUIRE(logits && work && temperature && top_p && uniform && out, "gl3_sample: null argument");
  GL3_REQUIRE(n_rows > 0 && V > 0 && ld >= V, "gl3_sample: bad sizes (rows=%d V=%d ld=%ld)", n_rows, V, ld);
  sample_kernel<<<dim3(n_rows), dim3(SB), 0, stream>>>(logits, ld, work, temperature, top_p, uniform, out, V, step,
                                                       uniform_stride);
  GL3_LAUNCH_CHECK();
  return 0;
}

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
// greatest threshold whose mass {p >= v} still exceeds top_p; v is found bit by
// bit over the float's pattern (31 passes), and the walk to the drawn token is the
// same search with u * mass in place of top_p. Masses are summed in 64-bit so that
// the order of the sum cannot move a comparison.
#include "common.h"

#define SB 1024

// inclusive scan of one double per thread over the block; result in cdf[SB]
__device__ void block_scan_f64(double v, double* cdf, double* wave_tot) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  double x = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    double y = __shfl_up(x, o, 64);
    if (lane >= o) x += y;
  }
  __syncthreads();
  if (lane == 63) wave_tot[wave] = x;
  __syncthreads();
  double off = 0.0;
  for (int w = 0; w < wave; ++w) off += wave_tot[w];
  cdf[threadIdx.x] = x + off;
  __syncthreads();
}

// greatest v (as a bit pattern) with sum{p_i >= v} > thr
__device__ uint32_t search_threshold(const float* p, int V, double thr, double* scratch) {
  uint32_t cur = 0;
  for (int bit = 30; bit >= 0; --bit) {
    const uint32_t cand = cur | (1u << bit);
    if (cand > 0x3f800000u) continue;  // above 1.0: no probability reaches it
    const float v = __uint_as_float(cand);
    double mass = 0.0;
    for (int i = threadIdx.x; i < V; i += SB) {
      const float pi = p[i];
      if (pi >= v) mass += (double)pi;
    }
    mass = block_sum_f64(mass, scratch);
    if (mass > thr) cur = cand;
  }
  return cur;
}

__global__ __launch_bounds__(SB) void sample_kernel(const float* __restrict__ logits, long ld, float* __restrict__ work,
                                                    const float* __restrict__ temperature,
                                                    const float* __restrict__ top_p, const float* __restrict__ uniform,
                                                    int* __restrict__ out, int V, const int* __restrict__ step,
                                                    int uniform_stride) {
  __shared__ float fs[16];
  __shared__ int is[16];
  __shared__ double ds[16];
  __shared__ double cdf[SB];
  __shared__ int winner;
  const int row = blockIdx.x, tid = threadIdx.x;
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

  float* p = work + (long)row * V;
  float m = -INFINITY;
  for (int i = tid; i < V; i += SB) m = fmaxf(m, lg[i] / T);
  m = block_max(m, fs);
  double z = 0.0;
  for (int i = tid; i < V; i += SB) {
    const float e = expf(lg[i] / T - m);
    p[i] = e;
    z += (double)e;
  }
  const float zf = (float)block_sum_f64(z, ds);
  for (int i = tid; i < V; i += SB) p[i] = p[i] / zf;
  __syncthreads();

  const float tp = top_p[row];
  // in a run of steps replayed from a graph the step's number is read from memory
  const double u = (double)uniform[(step ? (long)step[0] * uniform_stride : 0) + row];
  const int chunk = (V + SB - 1) / SB;
  const int b = min(V, tid * chunk), e = min(V, (tid + 1) * chunk);
  if (tid == 0) winner = -1;

  if (tp <= 0.f || tp >= 1.f) {
    double mine = 0.0;
    for (int i = b; i < e; ++i) mine += (double)p[i];
    block_scan_f64(mine, cdf, ds);
    const double before = tid ? cdf[tid - 1] : 0.0;
    if (before <= u && u < cdf[tid]) {
      double c = before;
      int pick = e - 1;
      for (int i = b; i < e; ++i) {
        c += (double)p[i];
        if (u < c) { pick = i; break; }
      }
      winner = pick;
    }
    __syncthreads();
    if (tid == 0) out[row] = winner >= 0 ? winner : V - 1;
    return;
  }

  // nucleus: threshold v1, the mass above it, and how many of the equal ones are kept
  const float v1 = __uint_as_float(search_threshold(p, V, (double)tp, ds));
  double gt = 0.0;
  for (int i = tid; i < V; i += SB) if (p[i] > v1) gt += (double)p[i];
  gt = block_sum_f64(gt, ds);
  double ties = 0.0;
  for (int i = tid; i < V; i += SB) if (p[i] == v1) ties += 1.0;
  ties = block_sum_f64(ties, ds);
  // smallest k >= 1 with gt + k * v1 > tp
  double k1 = v1 > 0.f ? floor(((double)tp - gt) / (double)v1) + 1.0 : ties;
  if (!(k1 >= 1.0)) k1 = 1.0;
  while (k1 > 1.0 && gt + (k1 - 1.0) * (double)v1 > (double)tp) k1 -= 1.0;
  while (k1 < ties && !(gt + k1 * (double)v1 > (double)tp)) k1 += 1.0;
  if (k1 > ties) k1 = ties;
  const double mass = gt + k1 * (double)v1;

  // the drawn token: first in the kept order whose running sum exceeds u * mass
  const double target = u * mass;
  const float v2 = __uint_as_float(search_threshold(p, V, target, ds));
  double gt2 = 0.0;
  for (int i = tid; i < V; i += SB) if (p[i] > v2) gt2 += (double)p[i];
  gt2 = block_sum_f64(gt2, ds);
  double ties2 = 0.0;
  for (int i = tid; i < V; i += SB) if (p[i] == v2) ties2 += 1.0;
  ties2 = block_sum_f64(ties2, ds);
  double j = v2 > 0.f ? floor((target - gt2) / (double)v2) : 0.0;
  if (!(j >= 0.0)) j = 0.0;
  while (j > 0.0 && target < gt2 + j * (double)v2) j -= 1.0;
  while (j + 1.0 < ties2 && !(target < gt2 + (j + 1.0) * (double)v2)) j += 1.0;
  double limit = ties2;
  if (v2 == v1) limit = k1;
  if (j > limit - 1.0) j = limit - 1.0;

  // the j-th (from 0) index in ascending order with p == v2
  double cnt = 0.0;
  for (int i = b; i < e; ++i) if (p[i] == v2) cnt += 1.0;
  block_scan_f64(cnt, cdf, ds);
  const double before = tid ? cdf[tid - 1] : 0.0;
  if (before <= j && j < cdf[tid]) {
    double c = before;
    for (int i = b; i < e; ++i)
      if (p[i] == v2) {
        if (c == j) { winner = i; break; }
        c += 1.0;
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

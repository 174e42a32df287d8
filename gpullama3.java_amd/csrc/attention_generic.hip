// Causal grouped-query attention over the paged cache for any head size up to
// 256, any number of heads and groups, float or bfloat16 storage, all arithmetic
// in 32-bit: the true 32-bit path and the fallback of the matrix-core kernels.
//
// One wave per (token, query head). Query head h reads kv head h / (H/K)
// (J/inference/InferenceCore.java:116-119). Keys lo..p are visited in chunks of 64
// that start at lo, one key per lane; score = dot(q, k) * scale with
// scale = 1/sqrt(head_dim) (:122); softmax with the running maximum
// (:128, FloatTensor.java:211-219 computes the same with the global maximum); the
// values are summed with the weights (:134-144). The chunking depends on the
// query's position alone, so a token's result is the same bit for bit whether it
// arrives with its whole prompt or alone.
#include "common.h"

#define ATT_MAX_HS 256

template <typename T>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const T* __restrict__ q, long q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int table_stride, T* __restrict__ out, long out_stride, int n_heads, int n_kv, int head_dim, int page_size,
    int window, float scale) {
  __shared__ float qs[ATT_MAX_HS];
  __shared__ float ps[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int p = positions[t];
  const int c = h / (n_heads / n_kv);
  const int* bt = block_table + (long)seq_of_token[t] * table_stride;
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const T* qp = q + (long)t * q_stride + (long)h * head_dim;
  for (int i = lane; i < head_dim; i += 64) qs[i] = to_f32<T>(qp[i]);
  __syncthreads();
  float m = -INFINITY, l = 0.f;
  float acc[ATT_MAX_HS / 64] = {};
  for (int base = lo; base <= p; base += 64) {
    const int key = base + lane;
    const bool valid = key <= p;
    float s = -INFINITY;
    if (valid) {
      const T* kp = k_cache + ((long)bt[key / page_size] * n_kv + c) * page_size * head_dim;
      const int in_page = key % page_size;
      float dot = 0.f;
      for (int i = 0; i < head_dim; ++i) dot = fmaf(qs[i], to_f32<T>(kp[gl3_k_offset(in_page, i, head_dim)]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pe = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(pe);
    __syncthreads();
    ps[lane] = pe;
    __syncthreads();
    const int n_valid = (p - base + 1 < 64) ? p - base + 1 : 64;
#pragma unroll
    for (int r = 0; r < ATT_MAX_HS / 64; ++r) acc[r] *= alpha;
    for (int j = 0; j < n_valid; ++j) {
      const int kj = base + j;
      // values lie transposed in a page: [head_dim][position in page], in tiles
      const T* vp = v_cache + ((long)bt[kj / page_size] * n_kv + c) * page_size * head_dim;
      const int in_page = kj % page_size;
      const float w = ps[j];
#pragma unroll
      for (int r = 0; r < ATT_MAX_HS / 64; ++r) {
        const int i = lane + 64 * r;
        if (i < head_dim) acc[r] = fmaf(w, to_f32<T>(vp[gl3_v_offset(i, in_page, page_size)]), acc[r]);
      }
    }
    m = m_new;
  }
  T* op = out + (long)t * out_stride + (long)h * head_dim;
#pragma unroll
  for (int r = 0; r < ATT_MAX_HS / 64; ++r) {
    const int i = lane + 64 * r;
    if (i < head_dim) op[i] = from_f32<T>(acc[r] / l);
  }
}

extern "C" int gl3_attention_generic(const void* q, long q_stride, const void* k_cache, const void* v_cache, int dtype,
                                     const int* positions, const int* seq_of_token, const int* block_table,
                                     int table_stride, void* out, long out_stride, int n_tokens, int n_heads, int n_kv,
                                     int head_dim, int page_size, int window, float scale, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(q && k_cache && v_cache && positions && seq_of_token && block_table && out,
              "gl3_attention_generic: null argument");
  GL3_REQUIRE(n_tokens > 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0,
              "gl3_attention_generic: %d heads over %d kv heads", n_heads, n_kv);
  GL3_REQUIRE(head_dim > 0 && head_dim <= ATT_MAX_HS, "gl3_attention_generic: head_dim %d exceeds %d", head_dim,
              ATT_MAX_HS);
  GL3_REQUIRE(n_heads <= 65535, "gl3_attention_generic: %d heads exceed the grid", n_heads);
  GL3_REQUIRE(page_size > 0 && table_stride > 0, "gl3_attention_generic: bad paging");
  GL3_REQUIRE(page_size % 32 == 0 && head_dim % 16 == 0,
              "gl3_attention_generic: the cache lies in tiles: page_size %d must be a multiple of 32, head_dim %d of 16", page_size,
              head_dim);
  dim3 grid(n_tokens, n_heads), block(64);
  if (dtype == GL3_F32)
    attention_generic_kernel<float><<<grid, block, 0, stream>>>(
        (const float*)q, q_stride, (const float*)k_cache, (const float*)v_cache, positions, seq_of_token, block_table,
        table_stride, (float*)out, out_stride, n_heads, n_kv, head_dim, page_size, window, scale);
  else if (dtype == GL3_BF16)
    attention_generic_kernel<bf16_t><<<grid, block, 0, stream>>>(
        (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, positions, seq_of_token,
        block_table, table_stride, (bf16_t*)out, out_stride, n_heads, n_kv, head_dim, page_size, window, scale);
  else GL3_REQUIRE(false, "gl3_attention_generic: unknown dtype %d", dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// Attention of a decode step in bfloat16: one new token per sequence against that
// sequence's keys and values in the paged cache. The time is the time to read the
// cache once, so keys and values go from memory straight into matrix-core operands.
//
// Formulas as J/inference/InferenceCore.java:106-145: score = q.k * scale over the keys
// lo..p, softmax, weighted sum of the values; query head h reads kv head h / (H/K).
//
// A block works on (token, kv head, group of up to 16 query heads, split of the key
// range); its four waves take chunks of 32 keys in turn. Per chunk, transposed:
//   S^T[key, head]  = K[key, :] . Q[head, :]^T      two 16x16 tiles, k = head_dim
//   O^T[dim, head] += V^T[dim, key] . P^T[key, head]  head_dim/16 tiles, k = 32 keys
// so a lane's 16 bytes of a key row, and of a row of the transposed value page, are the
// operands as the instruction wants them, and the probabilities leave the first
// product in the register order the second one takes (the 32 keys of a chunk are
// consumed in the order 4q..4q+3, 16+4q..16+4q+3 by both operands). Softmax keeps a
// running maximum and sum per head in 32-bit. The waves' partial results are merged
// in shared memory; with more than one split each block writes (max, sum, O) to a
// workspace and a second kernel merges the splits in split order.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int HS>
__global__ __launch_bounds__(256) void attention_decode_kernel(
    const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int table_stride, float* __restrict__ part_o, float* __restrict__ part_ml, bf16_t* __restrict__ out,
    long out_stride, int n_heads, int n_kv, int page_size, int window, float scale, int n_splits) {
  constexpr int KK = HS / 32;   // k-steps of the first product
  constexpr int DT = HS / 16;   // row tiles of the second product
  __shared__ float sm_m[4][16], sm_l[4][16];
  __shared__ f32x4 sm_o[4][DT][64];
  const int g = n_heads / n_kv;
  const int groups = (g + 15) / 16;
  const int t = blockIdx.x / (n_kv * groups);
  const int c = (blockIdx.x / groups) % n_kv;
  const int hg = blockIdx.x % groups;
  const int split = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int j = lane & 15, qd = lane >> 4;
  const int heads_here = min(16, g - hg * 16);
  const int h0 = c * g + hg * 16;

  const int kv_len = positions[t] + 1;
  const int lo = (window > 0 && kv_len > window) ? kv_len - window : 0;
  const int chunk_lo = lo / 32, chunk_hi = (kv_len + 31) / 32;
  const int per_split = (chunk_hi - chunk_lo + n_splits - 1) / n_splits;
  const int c_begin = chunk_lo + split * per_split;
  const int c_end = min(chunk_hi, c_begin + per_split);
  const int* bt = block_table + (long)seq_of_token[t] * table_stride;

  // Q^T operand: lane (head j, quarter qd) holds Q[h0 + j][kk*32 + 8*qd .. +7]
  bf16x8 qt[KK];
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int kk = 0; kk < KK; ++kk)
    qt[kk] = j < heads_here ? *(const bf16x8*)(q + (long)t * q_stride + (long)(h0 + j) * HS + kk * 32 + 8 * qd) : zero8;

  float m_run = -INFINITY, l_run = 0.f;   // l_run: this lane's share of the row sum
  f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int ck = c_begin + wave; ck < c_end; ck += 4) {
    const int key0 = ck * 32;
    const long page = bt[key0 / page_size];
    const int po = key0 % page_size;
    const bf16_t* kb = k_cache + ((page * n_kv + c) * page_size + po) * HS;
    const bf16_t* vb = v_cache + (page * n_kv + c) * (long)page_size * HS + po;
    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const bf16x8 ka = *(const bf16x8*)(kb + (long)j * HS + kk * 32 + 8 * qd);
      const bf16x8 kb2 = *(const bf16x8*)(kb + (long)(16 + j) * HS + kk * 32 + 8 * qd);
      sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qt[kk], sa, 0, 0, 0);
      sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb2, qt[kk], sb, 0, 0, 0);
    }
    // values: lane (dim i = j, quarter qd) takes keys 4qd..4qd+3 and 16+4qd..16+4qd+3 of the chunk
    bf16x8 vt[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const bf16_t* vr = vb + (long)(dt * 16 + j) * page_size + 4 * qd;
      const bf16x4 v0 = *(const bf16x4*)vr, v1 = *(const bf16x4*)(vr + 16);
      vt[dt] = bf16x8{v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
    }
    // lane (head j, quarter qd) holds scores of keys key0 + 4qd + v (sa) and key0 + 16 + 4qd + v (sb)
    float s[8];
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int ka_i = key0 + 4 * qd + v, kb_i = ka_i + 16;
      s[v] = (ka_i >= lo && ka_i < kv_len) ? sa[v] * scale : -INFINITY;
      s[4 + v] = (kb_i >= lo && kb_i < kv_len) ? sb[v] * scale : -INFINITY;
      mx = fmaxf(mx, fmaxf(s[v], s[4 + v]));
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __expf(m_run - m_use);   // m_run = -inf gives 0
    float ps = 0.f;
    bf16x8 pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float p = __expf(s[e] - m_use);
      ps += p;
      pb[e] = static_cast<bf16_t>(p);
    }
    l_run = l_run * alpha + ps;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      o[dt] *= alpha;
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[dt], pb, o[dt], 0, 0, 0);
    }
  }

  // merge the four waves
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if (qd == 0) { sm_m[wave][j] = m_run; sm_l[wave][j] = l_run; }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) sm_o[wave][dt][lane] = o[dt];
  __syncthreads();
  float M = sm_m[0][j];
#pragma unroll
  for (int w = 1; w < 4; ++w) M = fmaxf(M, sm_m[w][j]);
  float f[4], L = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = sm_m[w][j] == -INFINITY ? 0.f : __expf(sm_m[w][j] - M);
    L += f[w] * sm_l[w][j];
  }
  const int h = h0 + j;
  for (int dt = wave; dt < DT; dt += 4) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) acc += sm_o[w][dt][lane] * f[w];
    if (j >= heads_here) continue;
    const int dim = dt * 16 + 4 * qd;   // lane holds O^T[dim .. dim+3][head j]
    if (n_splits == 1) {
      bf16_t* op = out + (long)t * out_stride + (long)h * HS + dim;
      const float inv = 1.0f / L;
#pragma unroll
      for (int v = 0; v < 4; ++v) op[v] = static_cast<bf16_t>(acc[v] * inv);
    } else {
      *(f32x4*)(part_o + (((long)t * n_heads + h) * n_splits + split) * HS + dim) = acc;
    }
  }
  if (n_splits > 1 && wave == 0 && qd == 0 && j < heads_here) {
    float* ml = part_ml + (((long)t * n_heads + h) * n_splits + split) * 2;
    ml[0] = M;
    ml[1] = L;
  }
}

// Merge the splits of one (token, head): in split order, so the result has one order of summation.
__global__ void attention_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                              bf16_t* __restrict__ out, long out_stride, int n_heads, int head_dim,
                                              int n_splits) {
  const long th = blockIdx.x;   // token * n_heads + head
  const long t = th / n_heads, h = th % n_heads;
  const float* ml = part_ml + th * n_splits * 2;
  float M = -INFINITY;
  for (int s = 0; s < n_splits; ++s) M = fmaxf(M, ml[2 * s]);
  float L = 0.f;
  for (int s = 0; s < n_splits; ++s) L += (ml[2 * s] == -INFINITY ? 0.f : __expf(ml[2 * s] - M)) * ml[2 * s + 1];
  for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
    float acc = 0.f;
    for (int s = 0; s < n_splits; ++s) {
      const float f = ml[2 * s] == -INFINITY ? 0.f : __expf(ml[2 * s] - M);
      acc += f * part_o[(th * n_splits + s) * head_dim + d];
    }
    out[t * out_stride + h * head_dim + d] = static_cast<bf16_t>(acc / L);
  }
}

// Head sizes this kernel is built for; the caller takes the generic kernel otherwise.
extern "C" int gl3_attention_decode_supports(int head_dim, int page_size) {
  return (head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128) &&
         page_size % 32 == 0;
}

extern "C" int gl3_attention_decode(const void* q, long q_stride, const void* k_cache, const void* v_cache,
                                    const int* positions, const int* seq_of_token, const int* block_table,
                                    int table_stride, float* part_o, float* part_ml, long part_floats, void* out,
                                    long out_stride, int n_tokens, int n_heads, int n_kv, int head_dim, int page_size,
                                    int window, float scale, int n_splits, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(q && k_cache && v_cache && positions && seq_of_token && block_table && out,
              "gl3_attention_decode: null argument");
  GL3_REQUIRE(gl3_attention_decode_supports(head_dim, page_size),
              "gl3_attention_decode: head_dim %d / page_size %d is not built (32, 64, 96, 128; pages of a multiple of 32)",
              head_dim, page_size);
  GL3_REQUIRE(n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "gl3_attention_decode: %d heads over %d kv heads", n_heads,
              n_kv);
  GL3_REQUIRE(q_stride % 8 == 0 && (uintptr_t)q % 16 == 0, "gl3_attention_decode: queries must be 16-byte aligned");
  GL3_REQUIRE(n_splits >= 1 && n_splits <= 256, "gl3_attention_decode: n_splits=%d", n_splits);
  if (n_splits > 1)
    GL3_REQUIRE(part_o && part_ml && part_floats >= (long)n_tokens * n_heads * n_splits * (head_dim + 2),
                "gl3_attention_decode: workspace of %ld floats is too small", part_floats);
  const int groups = (n_heads / n_kv + 15) / 16;
  const long blocks = (long)n_tokens * n_kv * groups;
  GL3_REQUIRE(blocks < (1L << 31), "gl3_attention_decode: too many blocks");
  dim3 grid((unsigned)blocks, n_splits), block(256);
#define GO(HS)                                                                                                        \
  attention_decode_kernel<HS><<<grid, block, 0, stream>>>(                                                            \
      (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, positions, seq_of_token, block_table, \
      table_stride, part_o, part_ml, (bf16_t*)out, out_stride, n_heads, n_kv, page_size, window, scale, n_splits)
  switch (head_dim) {
    case 32: GO(32); break;
    case 64: GO(64); break;
    case 96: GO(96); break;
    default: GO(128); break;
  }
#undef GO
  GL3_LAUNCH_CHECK();
  if (n_splits > 1) {
    attention_decode_merge_kernel<<<dim3((unsigned)((long)n_tokens * n_heads)), dim3(64), 0, stream>>>(
        part_o, part_ml, (bf16_t*)out, out_stride, n_heads, head_dim, n_splits);
    GL3_LAUNCH_CHECK();
  }
  return 0;
}

// Embedding gather, RMSNorm and rotary encoding fused with the cache write.
// Statistics and rotation are computed in 32-bit whatever the storage type.
#include "common.h"

// ----------------------------------------------------------------- embedding
// out[t, :] = table[ids[t], :] as float (J/inference/InferenceCore.java:69); with `scale` != 1 the row
// is multiplied by it, with `pos_table` ([positions][d], the table's type) row positions[t] of it is
// added (the reference's model has neither: an embedding multiplier and learned absolute positions
// are what other decoders put here).
// ssq (may be null; then n_tokens <= 64): ssq[t] = sum of squares of row t, for a norm that is
// folded into the product that follows; with it next_weight [d] (float) and xg [n_tokens][d]
// (may be null): xg = bfloat16(next_weight * row), the rows as that product reads them.
template <typename TW, bool VEC>
__global__ void embed_kernel(const TW* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out, int d,
                             float* __restrict__ ssq, const float* __restrict__ next_weight, bf16_t* __restrict__ xg,
                             float scale, const TW* __restrict__ pos_table, const int* __restrict__ positions,
                             int operand_steps) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  // operand_steps > 0 (VEC only): the table is kept in the matrix operands' order alone (gl3_operand_offset)
  const TW* row = operand_steps ? table : table + (long)ids[t] * d;
  const long id = ids[t];
  const TW* prow = pos_table ? pos_table + (long)positions[t] * d : nullptr;
  float* o = out + t * d;
  float ss = 0.f;
  if (VEC) {
    // eight elements a thread and trip: a row of a decode step is one trip to memory, not eight
    typedef TW tw8 __attribute__((ext_vector_type(8)));
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    for (int i = threadIdx.x * 8; i < d; i += blockDim.x * 8) {
      const tw8 r8 = *(const tw8*)(row + (operand_steps ? gl3_operand_offset(id, i, operand_steps) : (long)i));
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = to_f32<TW>(r8[e]);
      if (scale != 1.0f) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= scale;
      }
      if (prow) {
        const tw8 p8 = *(const tw8*)(prow + i);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += to_f32<TW>(p8[e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
      *(f32x4*)(o + i) = f32x4{v[0], v[1], v[2], v[3]};
      *(f32x4*)(o + i + 4) = f32x4{v[4], v[5], v[6], v[7]};
      if (xg) {
        const f32x4 w0 = *(const f32x4*)(next_weight + i), w1 = *(const f32x4*)(next_weight + i + 4);
        bf16x8 g;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          g[e] = static_cast<bf16_t>(w0[e] * v[e]);
          g[4 + e] = static_cast<bf16_t>(w1[e] * v[4 + e]);
        }
        *(bf16x8*)(xg + t * d + i) = g;
      }
    }
  } else {
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
      float v = to_f32<TW>(row[i]);
      if (scale != 1.0f) v *= scale;
      if (prow) v += to_f32<TW>(prow[i]);
      o[i] = v;
      ss += v * v;
      if (xg) xg[t * d + i] = static_cast<bf16_t>(next_weight[i] * v);
    }
  }
  if (ssq) {
    ss = block_sum(ss, scratch);
    if (threadIdx.x == 0) ssq[t] = ss;
  }
}

extern "C" int gl3_embed(const void* table, int table_dtype, const int* ids, float* out, int n_tokens, int d,
                         float* ssq, const float* next_weight, void* xg, float scale, const void* pos_table,
                         const int* positions, int operand_steps, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(table && ids && out && n_tokens > 0 && d > 0, "gl3_embed: bad arguments (T=%d d=%d)", n_tokens, d);
  GL3_REQUIRE(!ssq || n_tokens <= 64, "gl3_embed: sums of squares are kept for at most 64 rows");
  GL3_REQUIRE((next_weight == nullptr) == (xg == nullptr) && (!xg || ssq),
              "gl3_embed: the next norm's weight and its rows come together, with the sums of squares");
  GL3_REQUIRE(!pos_table || positions, "gl3_embed: a table of positions needs the tokens' positions");
  dim3 grid(n_tokens), block(256);
  // 16-byte units where the rows allow them (a width of a multiple of 8, aligned bases)
  const bool vec = d % 8 == 0 && (uintptr_t)table % 32 == 0 && (uintptr_t)out % 16 == 0 &&
                   (!pos_table || (uintptr_t)pos_table % 32 == 0) &&
                   (!xg || ((uintptr_t)xg % 16 == 0 && (uintptr_t)next_weight % 16 == 0));
  // operand_steps > 0: the table lies in the matrix operands' order ([strip of 16 rows][k-step of 32][lane][8]) with
  // that many k-steps a strip; a row's 8 consecutive elements are still one 16-byte unit
  GL3_REQUIRE(operand_steps == 0 || (vec && operand_steps * 32 >= d),
              "gl3_embed: a table in the operands' order needs a width of a multiple of 8 and aligned rows");
#define GO(TW, VEC)                                                                                              \
  embed_kernel<TW, VEC><<<grid, block, 0, stream>>>((const TW*)table, ids, out, d, ssq, next_weight, (bf16_t*)xg, scale, \
                                                    (const TW*)pos_table, pos_table ? positions : nullptr, operand_steps)
  if (table_dtype == GL3_F32) { if (vec) GO(float, true); else GO(float, false); }
  else if (table_dtype == GL3_BF16) { if (vec) GO(bf16_t, true); else GO(bf16_t, false); }
  else GL3_REQUIRE(false, "gl3_embed: unknown dtype %d", table_dtype);
#undef GO
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- rmsnorm
// out[r, i] = w[i] * (ss * x[row(r), i]),  ss = 1/sqrt(mean(x^2) + eps)
// (J/inference/InferenceCore.java:47-56). One block per row; `rows` (may be
// null) picks the rows of x that are normalised, so that the final norm runs on
// the wanted positions only. The order of the sum depends on d alone.
// VEC 4 (rows of a multiple of 4 floats, 16-byte aligned): 16-byte loads, and a thread's first four
// elements stay in registers between the two passes, so rows of up to 4,096 floats are read once.
template <typename TW, typename TO, int VEC>
__global__ __launch_bounds__(1024) void rmsnorm_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                                       const TW* __restrict__ w, TO* __restrict__ out, int d, float eps) {
  typedef float vec_t __attribute__((ext_vector_type(VEC)));
  __shared__ float scratch[16];
  const long r = blockIdx.x;
  const long src = rows ? rows[r] : r;
  const float* xr = x + src * d;
  const int first = threadIdx.x * VEC, stride = blockDim.x * VEC;
  vec_t kept = vec_t(0.f);
  float ss = 0.f;
  for (int i = first; i < d; i += stride) {
    const vec_t v = *(const vec_t*)(xr + i);
    if (i == first) kept = v;
#pragma unroll
    for (int e = 0; e < VEC; ++e) ss += ((const float*)&v)[e] * ((const float*)&v)[e];
  }
  ss = block_sum(ss, scratch);
  ss = ss / (float)d;
  ss = ss + eps;
  ss = 1.0f / sqrtf(ss);
  TO* o = out + r * d;
  for (int i = first; i < d; i += stride) {
    const vec_t v = i == first ? kept : *(const vec_t*)(xr + i);
    typedef TO out_t __attribute__((ext_vector_type(VEC)));
    out_t res;
#pragma unroll
    for (int e = 0; e < VEC; ++e) res[e] = from_f32<TO>(to_f32<TW>(w[i + e]) * (ss * ((const float*)&v)[e]));
    *(out_t*)(o + i) = res;      // (VEC 4: the launcher has checked the output's alignment)
  }
}

extern "C" int gl3_rmsnorm(const float* x, const int* rows, const void* w, int w_dtype, void* out, int out_dtype,
                           int n_rows, int d, float eps, hipStream_t stream) {
  if (n_rows == 0) return 0;
  GL3_REQUIRE(x && w && out && n_rows > 0 && d > 0, "gl3_rmsnorm: bad arguments (rows=%d d=%d)", n_rows, d);
  const bool vec4 = d % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0;
  const int threads = !vec4 ? 256 : d / 4 >= 1024 ? 1024 : d / 4 > 256 ? 512 : 256;
  dim3 grid(n_rows), block(threads);
#define GO(TW, TO)                                                                                              \
  do {                                                                                                          \
    if (vec4) rmsnorm_kernel<TW, TO, 4><<<grid, block, 0, stream>>>(x, rows, (const TW*)w, (TO*)out, d, eps);   \
    else rmsnorm_kernel<TW, TO, 1><<<grid, block, 0, stream>>>(x, rows, (const TW*)w, (TO*)out, d, eps);        \
  } while (0)
  if (w_dtype == GL3_F32 && out_dtype == GL3_F32) GO(float, float);
  else if (w_dtype == GL3_F32 && out_dtype == GL3_BF16) GO(float, bf16_t);
  else if (w_dtype == GL3_BF16 && out_dtype == GL3_F32) GO(bf16_t, float);
  else if (w_dtype == GL3_BF16 && out_dtype == GL3_BF16) GO(bf16_t, bf16_t);
  else GL3_REQUIRE(false, "gl3_rmsnorm: unknown dtypes %d %d", w_dtype, out_dtype);
#undef GO
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- rows of the residual stream as they are
// out[r, i] = x[rows[r], i] in the activation type: what the head of a decoder without a final norm reads.
template <typename TO>
__global__ void gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ rows, TO* __restrict__ out, int d) {
  const long r = blockIdx.x;
  const float* xr = x + (long)rows[r] * d;
  TO* o = out + r * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = from_f32<TO>(xr[i]);
}

extern "C" int gl3_gather_rows(const float* x, const int* rows, void* out, int out_dtype, int n_rows, int d,
                               hipStream_t stream) {
  if (n_rows == 0) return 0;
  GL3_REQUIRE(x && rows && out && n_rows > 0 && d > 0, "gl3_gather_rows: bad arguments (rows=%d d=%d)", n_rows, d);
  if (out_dtype == GL3_F32) gather_rows_kernel<float><<<n_rows, 256, 0, stream>>>(x, rows, (float*)out, d);
  else if (out_dtype == GL3_BF16) gather_rows_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(x, rows, (bf16_t*)out, d);
  else GL3_REQUIRE(false, "gl3_gather_rows: unknown dtype %d", out_dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- slices of a product + rmsnorm
// A product whose K was cut into slices left its sums as P[slice][row][ldp] (float). Here they
// are added to the residual rows in slice order, x[row] += P[0][row] + P[1][row] + ..., and the
// rows' RMSNorm is written to `out` (null: the sums alone). With `rows` the listed rows are
// normalised and x is left as it was (a row may be listed twice). One block per row.
// A thread's first VEC elements stay in registers between the two passes, and the loads of up to
// eight slices are all asked for before the first is added: for rows of up to 4096 floats the
// kernel is two trips to memory.
template <typename TW, typename TO, int VEC>
__global__ __launch_bounds__(1024) void add_slices_rmsnorm_kernel(float* __restrict__ x, const int* __restrict__ rows,
                                                                  const float* __restrict__ P, int n_slices,
                                                                  long slice_stride, long ldp,
                                                                  const TW* __restrict__ w, TO* __restrict__ out, int d,
                                                                  float eps) {
  typedef float vec_t __attribute__((ext_vector_type(VEC)));
  __shared__ float scratch[16];
  const long r = blockIdx.x;
  const long src = rows ? rows[r] : r;
  float* xr = x + src * d;
  const float* pr = P + src * ldp;
  // the sum of the slices for elements i .. i+VEC-1, in slice order
  auto summed = [&](int i) {
    vec_t v = *(const vec_t*)(xr + i);
    for (int s0 = 0; s0 < n_slices; s0 += 8) {
      vec_t p[8];
#pragma unroll
      for (int s = 0; s < 8; ++s)
        p[s] = s0 + s < n_slices ? *(const vec_t*)(pr + (long)(s0 + s) * slice_stride + i) : vec_t(0.f);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < 8; ++s)
        if (s0 + s < n_slices) v += p[s];
    }
    return v;
  };
  const int first = threadIdx.x * VEC, stride = blockDim.x * VEC;
  vec_t kept = vec_t(0.f);
  float ss = 0.f;
  for (int i = first; i < d; i += stride) {
    const vec_t v = summed(i);
    if (i == first) kept = v;
    if (!rows) *(vec_t*)(xr + i) = v;
#pragma unroll
    for (int e = 0; e < VEC; ++e) ss += ((const float*)&v)[e] * ((const float*)&v)[e];
  }
  if (!out) return;
  ss = block_sum(ss, scratch);
  ss = ss / (float)d;
  ss = ss + eps;
  ss = 1.0f / sqrtf(ss);
  TO* o = out + r * d;
  for (int i = first; i < d; i += stride) {
    // beyond the kept elements: this thread's own stores, or the sum again when x was not written
    const vec_t v = i == first ? kept : (rows ? summed(i) : *(const vec_t*)(xr + i));
    typedef TO out_t __attribute__((ext_vector_type(VEC)));
    out_t res;
#pragma unroll
    for (int e = 0; e < VEC; ++e) res[e] = from_f32<TO>(to_f32<TW>(w[i + e]) * (ss * ((const float*)&v)[e]));
    *(out_t*)(o + i) = res;      // (VEC 4: the launcher has checked the output's alignment)
  }
}

extern "C" int gl3_add_slices_rmsnorm(float* x, const int* rows, const float* P, int n_slices, long slice_stride,
                                      long ldp, const void* w, int w_dtype, void* out, int out_dtype, int n_rows,
                                      int d, float eps, hipStream_t stream) {
  if (n_rows == 0) return 0;
  GL3_REQUIRE(x && P && n_rows > 0 && d > 0 && n_slices > 0 && ldp >= d,
              "gl3_add_slices_rmsnorm: bad arguments (rows=%d d=%d slices=%d)", n_rows, d, n_slices);
  GL3_REQUIRE((w != nullptr) == (out != nullptr), "gl3_add_slices_rmsnorm: weight and output come together");
  const bool vec4 = d % 4 == 0 && ldp % 4 == 0 && slice_stride % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)P % 16 == 0 &&
                    (uintptr_t)out % 16 == 0;
  const int per = vec4 ? 4 : 1;
  const int threads = d / per >= 1024 ? 1024 : d / per > 256 ? 512 : 256;
  dim3 grid(n_rows), block(threads);
#define GO(TW, TO)                                                                                              \
  do {                                                                                                          \
    if (vec4)                                                                                                   \
      add_slices_rmsnorm_kernel<TW, TO, 4><<<grid, block, 0, stream>>>(x, rows, P, n_slices, slice_stride, ldp, \
                                                                       (const TW*)w, (TO*)out, d, eps);         \
    else                                                                                                        \
      add_slices_rmsnorm_kernel<TW, TO, 1><<<grid, block, 0, stream>>>(x, rows, P, n_slices, slice_stride, ldp, \
                                                                       (const TW*)w, (TO*)out, d, eps);         \
  } while (0)
  if (!out) GO(float, float);
  else if (w_dtype == GL3_F32 && out_dtype == GL3_F32) GO(float, float);
  else if (w_dtype == GL3_F32 && out_dtype == GL3_BF16) GO(float, bf16_t);
  else if (w_dtype == GL3_BF16 && out_dtype == GL3_F32) GO(bf16_t, float);
  else if (w_dtype == GL3_BF16 && out_dtype == GL3_BF16) GO(bf16_t, bf16_t);
  else GL3_REQUIRE(false, "gl3_add_slices_rmsnorm: unknown dtypes %d %d", w_dtype, out_dtype);
#undef GO
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- rotary + cache write
// qkv[t] holds [n_heads q heads | n_kv k heads | n_kv v heads], each of head_dim.
// Queries are rotated in place; keys are rotated and written to the paged key
// cache, values are copied to the value cache (rotation before the write, so
// cached keys are already rotated: J/inference/InferenceCore.java:83-101).
// Pair j of a head is (2j, 2j+1) for adjacent pairing, (j, j + rot/2) for
// half pairing; the angle's cos and sin come from a table [position, rot/2]
// built on the host (J/inference/operation/RoPE.java:29-31). Elements beyond
// `rot_dim` pass through. A null table means no rotation at all.
// One layer's key cache is [page][kv head][position in page][head_dim]; its value cache
// is [page][kv head][head_dim][position in page]: values lie transposed, and inside a page
// both lie in tiles of 16 rows x 8 columns (gl3_k_offset, gl3_v_offset), which is the order in
// which the attention kernels' matrix-core products read them.
// The page of position p of sequence s is block_table[s * table_stride + p / page_size].
template <typename T>
__global__ void rope_cache_kernel(T* __restrict__ qkv, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                  const int* __restrict__ block_table, int table_stride, const float* __restrict__ cos_tab,
                                  const float* __restrict__ sin_tab, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                  int n_heads, int n_kv, int head_dim, int rot_dim, int adjacent, int page_size,
                                  int write_kv, long row_stride) {
  const int t = blockIdx.x;
  const int head = blockIdx.y;  // [0,H): q, [H,H+K): k, [H+K,H+2K): v
  const int pos = positions[t];
  const long row = (long)t * row_stride;
  T* src = qkv + row + (long)head * head_dim;
  const int half = rot_dim / 2;
  T* kpage = nullptr;      // a key head: its page; element i of the row goes to kpage[gl3_k_offset(in_page, i, head_dim)]
  const int in_page = pos % page_size;
  if (head >= n_heads) {
    if (!write_kv) return;
    const int c = (head - n_heads) % n_kv;
    const int page = block_table[(long)seq_of_token[t] * table_stride + pos / page_size];
    if (head >= n_heads + n_kv) {   // a value head: transposed, no rotation
      T* vpage = v_cache + ((long)page * n_kv + c) * page_size * head_dim;
      for (int i = threadIdx.x; i < head_dim; i += blockDim.x) vpage[gl3_v_offset(i, in_page, page_size)] = src[i];
      return;
    }
    kpage = k_cache + ((long)page * n_kv + c) * page_size * head_dim;
  }
  auto put = [&](int i, T v) {
    if (kpage) kpage[gl3_k_offset(in_page, i, head_dim)] = v;
    else src[i] = v;
  };
  const bool rotate = cos_tab != nullptr && head < n_heads + n_kv;
  if (!rotate) {
    if (kpage)
      for (int i = threadIdx.x; i < head_dim; i += blockDim.x) put(i, src[i]);
    return;
  }
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    const int i0 = adjacent ? 2 * j : j;
    const int i1 = adjacent ? 2 * j + 1 : j + half;
    const float c = cos_tab[(long)pos * half + j], s = sin_tab[(long)pos * half + j];
    const float v0 = to_f32<T>(src[i0]), v1 = to_f32<T>(src[i1]);
    put(i0, from_f32<T>(v0 * c - v1 * s));
    put(i1, from_f32<T>(v0 * s + v1 * c));
  }
  if (kpage)
    for (int i = rot_dim + threadIdx.x; i < head_dim; i += blockDim.x) put(i, src[i]);
}

// The same for bfloat16 rows in units of 8 elements (16 bytes): one block per token, a thread
// takes a unit of 8 pairs (half pairing: 8 elements and the 8 half a head further; adjacent
// pairing: 16 consecutive elements), of 8 elements that pass through, or of 8 elements of a value
// head. head_dim and rot_dim / 2 are multiples of 8.
typedef __bf16 rc_bf16x8 __attribute__((ext_vector_type(8)));
typedef float rc_f32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void rope_cache_vec_kernel(
    bf16_t* __restrict__ qkv, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const int* __restrict__ block_table, int table_stride, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int n_heads, int n_kv,
    int head_dim, int rot_dim, int adjacent, int page_size, int write_kv, long row_stride, int n_tokens) {
  // Blocks with consecutive numbers go to different XCDs, each with a second-level cache of its own; neighbouring
  // tokens go to one XCD. The values of 8 consecutive positions of a sequence share 16 bytes of a transposed page.
  // The first of the step's tokens in such a group of 8 positions writes the values of all of them that the step
  // brings (they follow it in the packed order): 16 bytes a dim where the group is whole, single elements at the
  // ends of a sequence's tokens. (One 2-byte store per token and dim before: a million partial writes a layer for
  // 2,048 tokens.)
  const int per_xcd = (n_tokens + 7) / 8;
  const int t = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (t >= n_tokens) return;
  const int pos = positions[t];
  bf16_t* row = qkv + (long)t * row_stride;
  const int half = rot_dim / 2;
  long page = 0;
  if (write_kv) page = block_table[(long)seq_of_token[t] * table_stride + pos / page_size];
  const int in_page = pos % page_size;
  const bool rotate = cos_tab != nullptr;
  const int rot_heads = write_kv ? n_heads + n_kv : n_heads;
  const int pair_units = rotate ? half / 8 : 0;              // per head
  const int plain_units = (head_dim - (rotate ? rot_dim : 0)) / 8;
  const int per_head = pair_units + plain_units;
  int v_units = 0, run = 0;                      // units of the value heads, and how many tokens' values this block writes
  if (write_kv) {
    const int seq = seq_of_token[t];
    const bool first = (pos & 7) == 0 || t == 0 || seq_of_token[t - 1] != seq || positions[t - 1] != pos - 1;
    if (first) {
      v_units = n_kv * (head_dim / 8);
      run = 1;
      while (run < 8 - (pos & 7) && t + run < n_tokens && seq_of_token[t + run] == seq && positions[t + run] == pos + run) ++run;
    }
  }
  const int total = rot_heads * per_head + v_units;
  for (int w = threadIdx.x; w < total; w += blockDim.x) {
    if (w >= rot_heads * per_head) {            // a unit of a value head: transposed into the cache
      const int u = w - rot_heads * per_head;
      const int ch = u / (head_dim / 8), e0 = (u % (head_dim / 8)) * 8;
      bf16_t* vpage = v_cache + ((long)page * n_kv + ch) * page_size * head_dim;
      const long at = gl3_v_offset(e0, in_page, page_size);   // dims e0 .. e0+7 lie in one tile, 8 elements apart
      const bf16_t* from = row + (long)(n_heads + n_kv + ch) * head_dim + e0;
      if (run == 8) {                            // a whole group of 8 positions (pos % 8 == 0): 16 bytes a dim
        rc_bf16x8 v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = *(const rc_bf16x8*)(from + (long)i * row_stride);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          rc_bf16x8 o;
#pragma unroll
          for (int i = 0; i < 8; ++i) o[i] = v[i][e];
          *(rc_bf16x8*)(vpage + at + 8 * e) = o;
        }
      } else {
        for (int i = 0; i < run; ++i) {
          const rc_bf16x8 v = *(const rc_bf16x8*)(from + (long)i * row_stride);
#pragma unroll
          for (int e = 0; e < 8; ++e) vpage[at + i + 8 * e] = v[e];
        }
      }
      continue;
    }
    const int head = w / per_head, u = w % per_head;
    bf16_t* src = row + (long)head * head_dim;
    bf16_t* kpage = head >= n_heads ? k_cache + ((long)page * n_kv + (head - n_heads)) * page_size * head_dim : nullptr;
    // where the 8 elements from e on go: back into the row (a query head) or into the key's page
    auto dst = [&](int e) { return kpage ? kpage + gl3_k_offset(in_page, e, head_dim) : src + e; };
    if (u >= pair_units) {                      // elements beyond the rotation pass through
      const int e0 = (rotate ? rot_dim : 0) + (u - pair_units) * 8;
      if (kpage) *(rc_bf16x8*)dst(e0) = *(const rc_bf16x8*)(src + e0);
      continue;
    }
    const int j0 = u * 8;                        // first of the unit's 8 pairs
    const float* cp = cos_tab + (long)pos * half + j0;
    const float* sp = sin_tab + (long)pos * half + j0;
    const rc_f32x4 c0 = *(const rc_f32x4*)cp, c1 = *(const rc_f32x4*)(cp + 4);
    const rc_f32x4 s0 = *(const rc_f32x4*)sp, s1 = *(const rc_f32x4*)(sp + 4);
    const int ea = adjacent ? 2 * j0 : j0, eb = adjacent ? 2 * j0 + 8 : j0 + half;
    const rc_bf16x8 a = *(const rc_bf16x8*)(src + ea), b = *(const rc_bf16x8*)(src + eb);
    rc_bf16x8 oa, ob;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float c = e < 4 ? c0[e] : c1[e - 4], sn = e < 4 ? s0[e] : s1[e - 4];
      // pair e of the unit: (a[e], b[e]) for half pairing; elements 2e, 2e+1 of the 16 for adjacent
      float v0, v1;
      if (adjacent) {
        v0 = e < 4 ? (float)a[2 * e] : (float)b[2 * e - 8];
        v1 = e < 4 ? (float)a[2 * e + 1] : (float)b[2 * e - 7];
      } else {
        v0 = (float)a[e];
        v1 = (float)b[e];
      }
      const bf16_t r0 = static_cast<bf16_t>(v0 * c - v1 * sn), r1 = static_cast<bf16_t>(v0 * sn + v1 * c);
      if (adjacent) {
        if (e < 4) { oa[2 * e] = r0; oa[2 * e + 1] = r1; }
        else { ob[2 * e - 8] = r0; ob[2 * e - 7] = r1; }
      } else {
        oa[e] = r0;
        ob[e] = r1;
      }
    }
    *(rc_bf16x8*)dst(ea) = oa;
    *(rc_bf16x8*)dst(eb) = ob;
  }
}

extern "C" int gl3_rope_cache_write(void* qkv, int dtype, const int* positions, const int* seq_of_token,
                                    const int* block_table, int table_stride, const float* cos_tab,
                                    const float* sin_tab, void* k_cache, void* v_cache, int n_tokens, int n_heads,
                                    int n_kv, int head_dim, int rot_dim, int adjacent, int page_size, int write_kv,
                                    hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(qkv && positions && n_tokens > 0 && n_heads > 0 && n_kv > 0 && head_dim > 0,
              "gl3_rope_cache_write: bad arguments");
  GL3_REQUIRE(rot_dim >= 0 && rot_dim <= head_dim && rot_dim % 2 == 0, "gl3_rope_cache_write: rot_dim %d of head_dim %d",
              rot_dim, head_dim);
  GL3_REQUIRE((cos_tab == nullptr) == (sin_tab == nullptr), "gl3_rope_cache_write: one table without the other");
  if (write_kv) {
    GL3_REQUIRE(k_cache && v_cache && block_table && seq_of_token && page_size > 0 && table_stride > 0,
                "gl3_rope_cache_write: cache arguments missing");
    GL3_REQUIRE(page_size % 32 == 0 && head_dim % 16 == 0,
                "gl3_rope_cache_write: the cache lies in tiles: page_size %d must be a multiple of 32, head_dim %d of 16",
                page_size, head_dim);
  }
  const int heads = write_kv ? n_heads + 2 * n_kv : n_heads;   // without the write a row holds queries only
  const long row_stride = (long)heads * head_dim;
  // bfloat16 rows whose sizes allow 16-byte units take the kernel of one block per token
  const bool units = dtype == GL3_BF16 && head_dim % 8 == 0 && rot_dim % 16 == 0 && (uintptr_t)qkv % 16 == 0 &&
                     (!cos_tab || ((uintptr_t)cos_tab % 16 == 0 && (uintptr_t)sin_tab % 16 == 0)) &&
                     (!write_kv || ((uintptr_t)k_cache % 16 == 0));
  if (units) {
    rope_cache_vec_kernel<<<dim3((n_tokens + 7) / 8 * 8), dim3(256), 0, stream>>>(
        (bf16_t*)qkv, positions, seq_of_token, block_table, table_stride, cos_tab, sin_tab, (bf16_t*)k_cache,
        (bf16_t*)v_cache, n_heads, n_kv, head_dim, cos_tab ? rot_dim : 0, adjacent, page_size, write_kv, row_stride, n_tokens);
    GL3_LAUNCH_CHECK();
    return 0;
  }
  GL3_REQUIRE(heads <= 65535, "gl3_rope_cache_write: %d heads exceed the grid", heads);
  dim3 grid(n_tokens, heads), block(64);
  if (dtype == GL3_F32)
    rope_cache_kernel<float><<<grid, block, 0, stream>>>((float*)qkv, positions, seq_of_token, block_table, table_stride,
                                                         cos_tab, sin_tab, (float*)k_cache, (float*)v_cache, n_heads, n_kv,
                                                         head_dim, rot_dim, adjacent, page_size, write_kv, row_stride);
  else if (dtype == GL3_BF16)
    rope_cache_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)qkv, positions, seq_of_token, block_table,
                                                          table_stride, cos_tab, sin_tab, (bf16_t*)k_cache,
                                                          (bf16_t*)v_cache, n_heads, n_kv, head_dim, rot_dim, adjacent,
                                                          page_size, write_kv, row_stride);
  else GL3_REQUIRE(false, "gl3_rope_cache_write: unknown dtype %d", dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- what hangs on a token's position
// A decode step's QKV products need, per token, the page its keys and values go to and its row of cos and sin:
// look-ups that wait for the token's position, a second trip to memory in each of them. They are the same for
// every layer that shares the block table and the rotation, so one small kernel makes them once per step:
// pages[t] = table[rows[t]][positions[t] / page_size]; rot[t] = cos[positions[t]] | sin[positions[t]] (half each);
// tables[t] (may be null) = the token's row of the block table up to its position's page, so that the attention of
// a decode step finds the pages of token t in row t, without the look-up of which row is the token's.
__global__ void token_facts_kernel(const int* __restrict__ positions, const int* __restrict__ rows,
                                   const int* __restrict__ block_table, int table_stride, int page_size,
                                   const float* __restrict__ cos_tab, const float* __restrict__ sin_tab, int half,
                                   int* __restrict__ pages, float* __restrict__ rot, int* __restrict__ tables) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int* row = block_table + (long)rows[t] * table_stride;
  if (threadIdx.x == 0) pages[t] = row[pos / page_size];
  if (tables)
    for (int j = threadIdx.x; j <= pos / page_size; j += blockDim.x) tables[(long)t * table_stride + j] = row[j];
  if (rot)
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
      rot[(long)t * 2 * half + j] = cos_tab[(long)pos * half + j];
      rot[(long)t * 2 * half + half + j] = sin_tab[(long)pos * half + j];
    }
}

// cos_tab, sin_tab, rot: all three or none (no rotation: the pages alone).
extern "C" int gl3_token_facts(const int* positions, const int* rows, const int* block_table, int table_stride,
                               int page_size, const float* cos_tab, const float* sin_tab, int half, int* pages, float* rot,
                               int* tables, int n_tokens, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(positions && rows && block_table && pages && table_stride > 0 && page_size > 0 && n_tokens > 0,
              "gl3_token_facts: bad arguments");
  GL3_REQUIRE((cos_tab != nullptr) == (sin_tab != nullptr) && (cos_tab != nullptr) == (rot != nullptr) && (!rot || half > 0),
              "gl3_token_facts: the tables and the rows for them come together");
  token_facts_kernel<<<dim3(n_tokens), dim3(64), 0, stream>>>(positions, rows, block_table, table_stride, page_size,
                                                              cos_tab, sin_tab, half, pages, rot, tables);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- between the steps of a run
// After a decode step whose tokens were sampled on the device: the sampled tokens become the next
// step's input, each sequence moves on by one position, the tokens are kept in a history row, and
// the step counter goes up. One block; n <= 1024.
__global__ void decode_advance_kernel(int* __restrict__ token_ids, int* __restrict__ positions,
                                      int* __restrict__ kv_before, const int* __restrict__ sampled,
                                      int* __restrict__ history, int history_stride, int* __restrict__ step, int n) {
  const int i = threadIdx.x;
  const int s = step[0];
  __syncthreads();
  if (i < n) {
    const int t = sampled[i];
    token_ids[i] = t;
    history[(long)s * history_stride + i] = t;
    positions[i] += 1;
    kv_before[i] += 1;
  }
  if (i == 0) step[0] = s + 1;
}

extern "C" int gl3_decode_advance(int* token_ids, int* positions, int* kv_before, const int* sampled, int* history,
                                  int history_stride, int* step, int n, hipStream_t stream) {
  GL3_REQUIRE(token_ids && positions && kv_before && sampled && history && step, "gl3_decode_advance: null argument");
  GL3_REQUIRE(n > 0 && n <= 1024 && history_stride >= n, "gl3_decode_advance: n=%d stride=%d", n, history_stride);
  decode_advance_kernel<<<dim3(1), dim3(1024), 0, stream>>>(token_ids, positions, kv_before, sampled, history,
                                                            history_stride, step, n);
  GL3_LAUNCH_CHECK();
  return 0;
}

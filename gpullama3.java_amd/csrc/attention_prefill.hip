// Causal grouped-query attention in bfloat16 for steps that bring many tokens per
// sequence (prompts, chunks), over the paged cache that already holds this step's keys
// and values. Formulas as J/inference/InferenceCore.java:106-145: query head h reads kv
// head h / (H/K); score = q.k * scale over the keys lo..p of the query's own position
// p; softmax; weighted sum of the values.
//
// A wave owns 16 consecutive queries of one sequence and up to GH query heads that
// share one kv head, so a key or value operand that it loads serves GH heads. It walks
// the keys in chunks of 32 with the running maximum and sum of the softmax in 32-bit.
// Both products are transposed, as in the decode kernel:
//   S^T[key, query]  = K[key, :] . Q[query, :]^T
//   O^T[dim, query] += V^T[dim, key] . P^T[key, query]
// which makes 16 bytes of a key row, and of a row of the transposed value page, the
// operands as the instruction wants them, and leaves the probabilities in the register
// order the second product takes (row i of the first score tile is key 8*(i/4) + i%4 of
// the chunk, row i of the second the key 4 further, so a quarter of the lanes ends up with
// 8 consecutive keys: one 16-byte load from a row of the transposed value page). The
// operands of the next chunk are asked for before the current chunk is worked on. The four
// waves of a block take neighbouring query tiles and share their keys and values through
// the caches only; they never wait for each other.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int HS, int GH>
__global__ __launch_bounds__(256) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ cu_seqlens, const int* __restrict__ kv_before, const int* __restrict__ block_table,
    int table_stride, bf16_t* __restrict__ out, long out_stride, int n_heads, int n_kv, int page_size, int window,
    float scale, int q_blocks) {
  constexpr int KK = HS / 32;
  constexpr int DT = HS / 16;
  const int g = n_heads / n_kv;
  const int groups = (g + GH - 1) / GH;
  // the longest query blocks first: blockIdx.x counts down through a sequence
  const int qb = q_blocks - 1 - blockIdx.x;
  const int b = blockIdx.y;
  const int c = blockIdx.z / groups, hg = blockIdx.z % groups;
  // scalar: what depends on the wave alone (chunk, page) lives in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int j = lane & 15, qd = lane >> 4;
  const int tok0 = __builtin_amdgcn_readfirstlane(cu_seqlens[b]);
  const int q_len = __builtin_amdgcn_readfirstlane(cu_seqlens[b + 1]) - tok0;
  const int qi0 = qb * 64 + wave * 16;   // first query of this wave, counted inside the step's tokens
  if (qi0 >= q_len) return;
  const int before = __builtin_amdgcn_readfirstlane(kv_before[b]);
  const int heads_here = min(GH, g - hg * GH);
  const int h0 = c * g + hg * GH;
  const int* bt = block_table + (long)b * table_stride;
  const bool q_ok = qi0 + j < q_len;
  const int p_mine = before + qi0 + j;                           // position of this lane's query
  const int p_last = before + min(qi0 + 15, q_len - 1);          // last position of the wave
  const int p_first = before + qi0;
  const int lo_first = (window > 0 && p_first + 1 > window) ? p_first + 1 - window : 0;
  const int lo_mine = (window > 0 && p_mine + 1 > window) ? p_mine + 1 - window : 0;

  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 qt[GH][KK];
#pragma unroll
  for (int hh = 0; hh < GH; ++hh)
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
      qt[hh][kk] = (q_ok && hh < heads_here)
                       ? *(const bf16x8*)(q + (long)(tok0 + qi0 + j) * q_stride + (long)(h0 + hh) * HS + kk * 32 + 8 * qd)
                       : zero8;

  float m_run[GH], l_run[GH];
  f32x4 o[GH][DT];
#pragma unroll
  for (int hh = 0; hh < GH; ++hh) {
    m_run[hh] = -INFINITY;
    l_run[hh] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[hh][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int krow = 8 * (j >> 2) + (j & 3);   // which key of a chunk is row j of the first score tile
  bf16x8 ka[KK], kb2[KK], vt[DT], ka_n[KK], kb2_n[KK], vt_n[DT];
  auto load_chunk = [&](int ck, bf16x8 (&a)[KK], bf16x8 (&b2)[KK], bf16x8 (&v)[DT]) {
    const int key0 = ck * 32;
    const long page = __builtin_amdgcn_readfirstlane(bt[key0 / page_size]);
    const int po = key0 % page_size;
    const bf16_t* kb = k_cache + ((page * n_kv + c) * page_size + po) * HS;
    const bf16_t* vb = v_cache + (page * n_kv + c) * (long)page_size * HS + po;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      a[kk] = *(const bf16x8*)(kb + (long)krow * HS + kk * 32 + 8 * qd);
      b2[kk] = *(const bf16x8*)(kb + (long)(krow + 4) * HS + kk * 32 + 8 * qd);
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) v[dt] = *(const bf16x8*)(vb + (long)(dt * 16 + j) * page_size + 8 * qd);
  };
  const int ck_first = lo_first / 32, ck_last = p_last / 32;
  load_chunk(ck_first, ka, kb2, vt);
  for (int ck = ck_first; ck <= ck_last; ++ck) {
    const int key0 = ck * 32;
    if (ck < ck_last) load_chunk(ck + 1, ka_n, kb2_n, vt_n);   // on its way while this chunk is worked on
    __builtin_amdgcn_sched_barrier(0);
    // this lane's 8 keys of the chunk and whether its query may see them
    bool see[8];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int k1 = key0 + 8 * qd + v, k2 = k1 + 4;
      see[v] = k1 >= lo_mine && k1 <= p_mine;
      see[4 + v] = k2 >= lo_mine && k2 <= p_mine;
    }
#pragma unroll
    for (int hh = 0; hh < GH; ++hh) {
      f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kk], qt[hh][kk], sa, 0, 0, 0);
        sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb2[kk], qt[hh][kk], sb, 0, 0, 0);
      }
      float s[8];
      float mx = -INFINITY;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        s[v] = see[v] ? sa[v] * scale : -INFINITY;
        s[4 + v] = see[4 + v] ? sb[v] * scale : -INFINITY;
        mx = fmaxf(mx, fmaxf(s[v], s[4 + v]));
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run[hh], mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __expf(m_run[hh] - m_use);
      float ps = 0.f;
      bf16x8 pb;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __expf(s[e] - m_use);
        ps += p;
        pb[e] = static_cast<bf16_t>(p);
      }
      l_run[hh] = l_run[hh] * alpha + ps;
      m_run[hh] = m_new;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        o[hh][dt] *= alpha;
        o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[dt], pb, o[hh][dt], 0, 0, 0);
      }
    }
    if (ck < ck_last) {
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) { ka[kk] = ka_n[kk]; kb2[kk] = kb2_n[kk]; }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) vt[dt] = vt_n[dt];
    }
  }

#pragma unroll
  for (int hh = 0; hh < GH; ++hh) {
    float l = l_run[hh];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!q_ok || hh >= heads_here) continue;
    const float inv = 1.0f / l;
    bf16_t* op = out + (long)(tok0 + qi0 + j) * out_stride + (long)(h0 + hh) * HS + 4 * qd;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      bf16x4 r;
#pragma unroll
      for (int v = 0; v < 4; ++v) r[v] = static_cast<bf16_t>(o[hh][dt][v] * inv);
      *(bf16x4*)(op + dt * 16) = r;
    }
  }
}

extern "C" int gl3_attention_prefill_supports(int head_dim, int page_size) {
  return (head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128) && page_size % 32 == 0;
}

// max_q_len: the most tokens any sequence brings in this step (it sizes the grid).
extern "C" int gl3_attention_prefill(const void* q, long q_stride, const void* k_cache, const void* v_cache,
                                     const int* cu_seqlens, const int* kv_before, const int* block_table,
                                     int table_stride, void* out, long out_stride, int n_seqs, int max_q_len,
                                     int n_heads, int n_kv, int head_dim, int page_size, int window, float scale,
                                     hipStream_t stream) {
  if (n_seqs == 0 || max_q_len == 0) return 0;
  GL3_REQUIRE(q && k_cache && v_cache && cu_seqlens && kv_before && block_table && out,
              "gl3_attention_prefill: null argument");
  GL3_REQUIRE(gl3_attention_prefill_supports(head_dim, page_size),
              "gl3_attention_prefill: head_dim %d / page_size %d is not built (32, 64, 96, 128; pages of a multiple of 32)",
              head_dim, page_size);
  GL3_REQUIRE(n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "gl3_attention_prefill: %d heads over %d kv heads",
              n_heads, n_kv);
  GL3_REQUIRE(q_stride % 8 == 0 && (uintptr_t)q % 16 == 0 && out_stride % 4 == 0 && (uintptr_t)out % 8 == 0,
              "gl3_attention_prefill: queries must be 16-byte aligned, outputs 8-byte aligned");
  const int g = n_heads / n_kv;
  const int q_blocks = (max_q_len + 63) / 64;
  const int gh = head_dim > 64 ? 2 : 4;
  const long z = (long)n_kv * ((g + gh - 1) / gh);
  GL3_REQUIRE(n_seqs <= 65535 && z <= 65535, "gl3_attention_prefill: %d sequences / %ld head groups exceed the grid",
              n_seqs, z);
  dim3 grid(q_blocks, n_seqs, (unsigned)z), block(256);
#define GO(HS, GH)                                                                                                  \
  attention_prefill_kernel<HS, GH><<<grid, block, 0, stream>>>(                                                     \
      (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, cu_seqlens, kv_before, block_table, \
      table_stride, (bf16_t*)out, out_stride, n_heads, n_kv, page_size, window, scale, q_blocks)
  switch (head_dim) {
    case 32: GO(32, 4); break;
    case 64: GO(64, 4); break;
    case 96: GO(96, 2); break;
    default: GO(128, 2); break;
  }
#undef GO
  GL3_LAUNCH_CHECK();
  return 0;
}

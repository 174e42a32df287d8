// Attention of a decode step in bfloat16: one new token per sequence against that
// sequence's keys and values in the paged cache. The time is the time to read the
// cache once, so keys and values go from memory straight into matrix-core operands.
//
// Formulas as J/inference/InferenceCore.java:106-145: score = q.k * scale over the keys
// lo..p, softmax, weighted sum of the values; query head h reads kv head h / (H/K).
//
// A block works on (token, kv head, group of up to 16 query heads, split of the key
// range); its NW waves take chunks of 32 keys in turn, and a wave asks for the keys and
// values of CB chunks at once before it works on the first: the work per chunk is short
// next to a trip to memory, so the trips must overlap. (Asking for the chunk CB places on as
// soon as one has been worked on, so that loads are on their way during the work too, was no
// faster at any context and 2.5% slower at 32,768 keys.) Per chunk, transposed:
//   S^T[key, head]  = K[key, :] . Q[head, :]^T      two 16x16 tiles, k = head_dim
//   O^T[dim, head] += V^T[dim, key] . P^T[key, head]  head_dim/16 tiles, k = 32 keys
// so a lane's 16 bytes of a key row, and of a row of the transposed value page, are the
// operands as the instruction wants them (and the cache keeps a page in tiles, gl3_k_offset and
// gl3_v_offset, in which a wave's operand is 1 KB of consecutive memory: with plain rows every
// lane of a load touched a line of its own, and a chunk's eight loads kept a CU's first-level
// cache busy for a quarter of the kernel's time), and the probabilities leave the first
// product in the register order the second one takes: row i of the first score tile is
// key 8*(i/4) + i%4 of the chunk and row i of the second is the key 4 further, so that
// quarter q of the lanes ends up with keys 8q..8q+7, which is one 16-byte load from a
// row of the transposed value page. Softmax keeps a
// running maximum and sum per head in 32-bit. The waves' partial results are merged
// in shared memory (heads of more than 64: the upper half of the waves hands its results to
// the lower half first, so that eight waves' results need the room of four: with four waves a
// context of 560 keys took three trips to memory one after the other, with eight it takes
// two, of which the second is nearly empty); with more than one split each block writes
// (max, sum, O) to a workspace and a second kernel merges the splits in split order.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Time stamps inside the kernel, for measurements (compiled in with -DAD_STAMPS only, never in the library's own build).
#ifdef AD_STAMPS
__device__ long long ad_stamps[2][2][16];
extern "C" int gl3_ad_stamps(long long* out) {
  return hipMemcpyFromSymbol(out, HIP_SYMBOL(ad_stamps), sizeof(ad_stamps)) == hipSuccess ? 0 : -1;
}
#define AD_STAMP(i)                                                                                              \
  do {                                                                                                           \
    const int w_ = threadIdx.x >> 6, nw_ = blockDim.x >> 6;                                                      \
    if ((blockIdx.x == 0 || blockIdx.x == gridDim.x / 2) && (threadIdx.x & 63) == 0 && (w_ == 0 || w_ == nw_ - 1)) \
      ad_stamps[blockIdx.x == 0 ? 0 : 1][w_ == 0 ? 0 : 1][i] = (i) == 0 || (i) == 15 ? wall_clock64() : clock64(); \
  } while (0)
#else
#define AD_STAMP(i) do {} while (0)
#endif

// P2: a page holds a power of two of positions (page_size == 1 << page_shift): a chunk's page and its place in it are
// a shift and a mask. A division by a number only known at run time is some forty scalar instructions, and the
// kernel has eight of them in front of its first loads.
template <int HS, int NW, int CB, bool P2>
__global__ __launch_bounds__(NW * 64) void attention_decode_kernel(
    const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int table_stride, float* __restrict__ part_o, float* __restrict__ part_ml, bf16_t* __restrict__ out,
    long out_stride, int n_heads, int n_kv, int g, int page_size, int page_shift, int window, float scale, int n_splits) {
  constexpr int KK = HS / 32;   // k-steps of the first product
  constexpr int DT = HS / 16;   // row tiles of the second product
  constexpr int NS = (HS > 64 && NW > 4) ? NW / 2 : NW;   // partial results that shared memory holds at a time
  __shared__ float sm_m[NS][16], sm_l[NS][16];
  __shared__ f32x4 sm_o[NS][DT][64];
  AD_STAMP(0); AD_STAMP(1);
  // the grid: (kv head and group of 16 query heads, split, token)
  // (g = n_heads / n_kv comes from the host: the division would stand in front of everything else)
  const int groups = (g + 15) / 16;
  const int t = blockIdx.z;
  const int c = groups == 1 ? (int)blockIdx.x : (int)blockIdx.x / groups;
  const int hg = groups == 1 ? 0 : (int)blockIdx.x % groups;
  const int split = blockIdx.y;
  auto page_of = [&](int key) { return P2 ? key >> page_shift : key / page_size; };
  auto in_page = [&](int key) { return P2 ? key & (page_size - 1) : key % page_size; };
  // the wave's number as a scalar: what depends on it alone (chunk, page) then lives in scalar
  // registers and its table look-ups are scalar loads, not a trip to memory per lane
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int j = lane & 15, qd = lane >> 4;
  const int heads_here = min(16, g - hg * 16);
  const int h0 = c * g + hg * 16;

  // The token's row of the block table: row seq_of_token[t], or (seq_of_token null) row t of a table that the step
  // made of its own tokens' rows. Then nothing stands between the kernel's start and the page numbers: those of the
  // chunks that this wave would take first in a sequence read from its start (no window, one split: every decode
  // step of a short context) are asked for together with the token's position, one trip to memory instead of two.
  const int* bt = block_table + (long)(seq_of_token ? __builtin_amdgcn_readfirstlane(seq_of_token[t]) : t) * table_stride;
  int first_pages[CB];
#pragma unroll
  for (int b = 0; b < CB; ++b)
    first_pages[b] = __builtin_amdgcn_readfirstlane(bt[min(page_of((wave + b * NW) * 32), table_stride - 1)]);
  const int kv_len = __builtin_amdgcn_readfirstlane(positions[t]) + 1;
  const int lo = (window > 0 && kv_len > window) ? kv_len - window : 0;
  const int chunk_lo = lo / 32, chunk_hi = (kv_len + 31) / 32;
  const int per_split = n_splits == 1 ? chunk_hi - chunk_lo : (chunk_hi - chunk_lo + n_splits - 1) / n_splits;
  const int c_begin = chunk_lo + split * per_split;
  const int c_end = min(chunk_hi, c_begin + per_split);
  AD_STAMP(2);

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

  for (int ck0 = c_begin + wave; ck0 < c_end; ck0 += NW * CB) {
    // operands of CB chunks, all asked for before any is used
    bf16x8 ka[CB][KK], kb2[CB][KK], vt[CB][DT];
#pragma unroll
    for (int b = 0; b < CB; ++b) {
      const int ck = ck0 + b * NW;
      if (ck < c_end) {
        const int key0 = ck * 32;
        // (the first chunks from the sequence's start: their pages are here already)
        const long page = (c_begin == 0 && ck0 == wave) ? first_pages[b] : __builtin_amdgcn_readfirstlane(bt[page_of(key0)]);
        const int po = in_page(key0);
        // the chunk's two key tiles lie one after the other, 16 * HS elements each; a k-step's operand
        // is 512 consecutive elements of a tile in lane order (gl3_k_offset)
        const bf16_t* kb = k_cache + ((page * n_kv + c) * page_size + po) * HS + lane * 8;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          ka[b][kk] = *(const bf16x8*)(kb + kk * 512);
          kb2[b][kk] = *(const bf16x8*)(kb + 16 * HS + kk * 512);
        }
        // values: lane (dim j of the tile, quarter qd) takes keys 8qd..8qd+7 of the chunk: 512
        // consecutive elements of the tile row of 16 dims (gl3_v_offset)
        const bf16_t* vb = v_cache + (page * n_kv + c) * (long)page_size * HS + (long)(po / 8) * 128 + lane * 8;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vt[b][dt] = *(const bf16x8*)(vb + (long)dt * page_size * 16);
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // every load above is issued before the first is waited for
    AD_STAMP(3);
#pragma unroll
    for (int b = 0; b < CB; ++b) {
      const int ck = ck0 + b * NW;
      if (ck >= c_end) break;
      const int key0 = ck * 32;
      f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[b][kk], qt[kk], sa, 0, 0, 0);
        sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb2[b][kk], qt[kk], sb, 0, 0, 0);
      }
      // lane (head j, quarter qd) holds scores of keys key0 + 8qd + v (sa) and key0 + 8qd + 4 + v (sb)
      float s[8];
      float mx = -INFINITY;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int ka_i = key0 + 8 * qd + v, kb_i = ka_i + 4;
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
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[b][dt], pb, o[dt], 0, 0, 0);
      }
    }
  }

#ifdef AD_STAMPS
  asm volatile("s_nop 0" :: "v"(o[0][0]));
  AD_STAMP(4);
#endif
  // merge the waves, in wave order
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if (NS < NW) {
    // wave w + NS hands its results to wave w, which then stands for both
    if (wave >= NS) {
      if (qd == 0) { sm_m[wave - NS][j] = m_run; sm_l[wave - NS][j] = l_run; }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) sm_o[wave - NS][dt][lane] = o[dt];
    }
    __syncthreads();
    if (wave < NS) {
      const float m2 = sm_m[wave][j], l2 = sm_l[wave][j];
      const float m_new = fmaxf(m_run, m2);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float f1 = __expf(m_run - m_use), f2 = __expf(m2 - m_use);   // a maximum of -inf gives 0
      l_run = l_run * f1 + l2 * f2;
      m_run = m_new;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[dt] = o[dt] * f1 + sm_o[wave][dt][lane] * f2;
    }
    __syncthreads();
  }
  if (wave < NS) {
    if (qd == 0) { sm_m[wave][j] = m_run; sm_l[wave][j] = l_run; }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) sm_o[wave][dt][lane] = o[dt];
  }
  __syncthreads();
  AD_STAMP(5);
  float M = sm_m[0][j];
#pragma unroll
  for (int w = 1; w < NS; ++w) M = fmaxf(M, sm_m[w][j]);
  float f[NS], L = 0.f;
#pragma unroll
  for (int w = 0; w < NS; ++w) {
    f[w] = sm_m[w][j] == -INFINITY ? 0.f : __expf(sm_m[w][j] - M);
    L += f[w] * sm_l[w][j];
  }
  const int h = h0 + j;
  for (int dt = wave; dt < DT; dt += NW) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < NS; ++w) acc += sm_o[w][dt][lane] * f[w];
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
  AD_STAMP(9); AD_STAMP(15);
}

// Merge the splits of one (token, head); one wave. Lane i holds the maxima and sums of splits i, i + 64, ...
// (all on their way at once; read one after the other, sixteen splits took 11 us), the factors go from
// lane to lane, and every lane adds up its dims over the splits in split order, eight splits' loads at a time.
__global__ __launch_bounds__(64) void attention_decode_merge_kernel(const float* __restrict__ part_o,
                                                                    const float* __restrict__ part_ml,
                                                                    bf16_t* __restrict__ out, long out_stride, int n_heads,
                                                                    int head_dim, int n_splits) {
  const long th = blockIdx.x;   // token * n_heads + head
  const long t = th / n_heads, h = th % n_heads;
  const int lane = threadIdx.x;
  const float* ml = part_ml + th * n_splits * 2;
  float m[4], l[4];             // (at most 256 splits)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int sp = lane + 64 * i;
    m[i] = sp < n_splits ? ml[2 * sp] : -INFINITY;
    l[i] = sp < n_splits ? ml[2 * sp + 1] : 0.f;
  }
  float M = fmaxf(fmaxf(m[0], m[1]), fmaxf(m[2], m[3]));
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) M = fmaxf(M, __shfl_xor(M, d, 64));
  float f[4], L = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[i] = m[i] == -INFINITY ? 0.f : __expf(m[i] - M);
    L += f[i] * l[i];
  }
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) L += __shfl_xor(L, d, 64);
  const float* po = part_o + th * n_splits * head_dim;
  for (int d = lane; d < head_dim + lane; d += 64) {     // (every lane walks the same number of times: the factors travel between lanes)
    const bool mine = d < head_dim;
    float acc = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += 8) {
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (mine && s0 + e < n_splits) ? po[(long)(s0 + e) * head_dim + d] : 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int sp = s0 + e;   // (the same for all lanes)
        const float fs = __shfl(sp < 64 ? f[0] : sp < 128 ? f[1] : sp < 192 ? f[2] : f[3], sp & 63, 64);
        acc += fs * v[e];
      }
    }
    if (mine) out[t * out_stride + h * head_dim + d] = static_cast<bf16_t>(acc / L);
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
  GL3_REQUIRE(q && k_cache && v_cache && positions && block_table && out && table_stride > 0,
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
  GL3_REQUIRE((long)n_kv * groups < (1L << 31) && n_tokens <= 65535, "gl3_attention_decode: too many blocks (%d tokens)", n_tokens);
  dim3 grid((unsigned)(n_kv * groups), n_splits, n_tokens);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  const bool p2 = (1 << page_shift) == page_size;
  // 8 waves; as many chunks on their way per wave as the registers hold (two waves share a SIMD's registers).
  // More blocks than CUs: 4 waves, so that a CU holds two blocks and the second 256 blocks do not wait for the
  // first to end (what a block does before its keys arrive is a chain of trips to memory, paid once per round).
  const bool small = blocks * n_splits > 256;
#define AD_ARGS                                                                                                       \
  (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, positions, seq_of_token, block_table,    \
      table_stride, part_o, part_ml, (bf16_t*)out, out_stride, n_heads, n_kv, n_heads / n_kv, page_size, page_shift, window,  \
      scale, n_splits
#define GO(HS)                                                                                                        \
  do {                                                                                                                \
    constexpr int CB = HS <= 64 ? 4 : HS <= 96 ? 3 : 2;                                                               \
    if (small && p2) attention_decode_kernel<HS, 4, CB, true><<<grid, dim3(256), 0, stream>>>(AD_ARGS);                \
    else if (small) attention_decode_kernel<HS, 4, CB, false><<<grid, dim3(256), 0, stream>>>(AD_ARGS);                \
    else if (p2) attention_decode_kernel<HS, 8, CB, true><<<grid, dim3(512), 0, stream>>>(AD_ARGS);                    \
    else attention_decode_kernel<HS, 8, CB, false><<<grid, dim3(512), 0, stream>>>(AD_ARGS);                           \
  } while (0)
  switch (head_dim) {
    case 32: GO(32); break;
    case 64: GO(64); break;
    case 96: GO(96); break;
    default: GO(128); break;
  }
#undef GO
#undef AD_ARGS
  GL3_LAUNCH_CHECK();
  if (n_splits > 1) {
    attention_decode_merge_kernel<<<dim3((unsigned)((long)n_tokens * n_heads)), dim3(64), 0, stream>>>(
        part_o, part_ml, (bf16_t*)out, out_stride, n_heads, head_dim, n_splits);
    GL3_LAUNCH_CHECK();
  }
  return 0;
}

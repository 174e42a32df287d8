// Causal grouped-query attention in bfloat16 for steps that bring many tokens per
// sequence (prompts, chunks), over the paged cache that already holds this step's keys
// and values. Formulas as J/inference/InferenceCore.java:106-145: query head h reads kv
// head h / (H/K); score = q.k * scale over the keys lo..p of the query's own position
// p; softmax; weighted sum of the values.
//
// A block is four waves on 64 consecutive queries of one sequence; a wave owns 16 of them
// and up to GH query heads that share one kv head. The block walks the keys in chunks of
// 32: its 256 threads bring a chunk of keys and of transposed values from the cache into
// shared memory once (the next chunk travels to registers while the current one is
// worked on, and goes into the other of two buffers), and every wave reads its operands
// from there, so the first-level cache carries each key once per block and not once per
// wave. Both products are transposed, as in the decode kernel:
//   S^T[key, query]  = K[key, :] . Q[query, :]^T
//   O^T[dim, query] += V^T[dim, key] . P^T[key, query]
// which makes 16 bytes of a key row, and of a row of the transposed value page, the
// operands as the instruction wants them, and leaves the probabilities in the register
// order the second product takes (row i of the first score tile is key 8*(i/4) + i%4 of
// the chunk, row i of the second the key 4 further, so a quarter of the lanes ends up with
// 8 consecutive keys). The running maximum and sum of the softmax are kept in 32-bit, in
// units of log2: p = 2^(s*scale*log2(e) - m) is one multiply-add and one exponential per
// score; chunks that every query of the wave sees whole skip the mask, and the sums are
// rescaled only when some maximum moved. Rows in shared memory are padded by 16 bytes, which
// spreads the 16 rows that a quarter of the lanes reads over all banks.
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// max over the four lanes j, j+16, j+32, j+48 (which hold different keys of one query), by the
// row-swap instructions: no trip through shared memory as a general shuffle makes
__device__ __forceinline__ float max_over_quarters(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  const float m = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(m), __float_as_uint(m), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

template <int HS, int GH>
__global__ __launch_bounds__(256, 2) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ cu_seqlens, const int* __restrict__ kv_before, const int* __restrict__ block_table,
    const int* __restrict__ seq_rows, int table_stride, bf16_t* __restrict__ out, long out_stride, int n_heads, int n_kv, int page_size, int window,
    float scale, int q_blocks) {
  constexpr int KK = HS / 32;
  constexpr int DT = HS / 16;
  constexpr int KROW = HS + 8;            // a key row in shared memory, in elements
  constexpr int VROW = 32 + 8;            // a row of the transposed value chunk
  constexpr int UNITS = HS * 4;           // 16-byte units of a chunk of keys (and of values)
  constexpr int NU = (UNITS + 255) / 256; // units per thread
  __shared__ __attribute__((aligned(16))) bf16_t ks[2][32][KROW];
  __shared__ __attribute__((aligned(16))) bf16_t vs[2][HS][VROW];
  const int g = n_heads / n_kv;
  const int groups = (g + GH - 1) / GH;
  // the longest query blocks first, of all heads and sequences: blockIdx.z counts down through a
  // sequence, the heads (x, which varies fastest as blocks are handed out) and sequences inside it
  const int qb = q_blocks - 1 - blockIdx.z;
  const int b = blockIdx.y;
  const int c = blockIdx.x / groups, hg = blockIdx.x % groups;
  // scalar: what depends on the wave alone (chunk, page) lives in scalar registers
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int j = lane & 15, qd = lane >> 4;
  const int tok0 = __builtin_amdgcn_readfirstlane(cu_seqlens[b]);
  const int q_len = __builtin_amdgcn_readfirstlane(cu_seqlens[b + 1]) - tok0;
  if (qb * 64 >= q_len) return;            // the whole block: no barrier has been passed yet
  const int before = __builtin_amdgcn_readfirstlane(kv_before[b]);
  const int heads_here = min(GH, g - hg * GH);
  const int h0 = c * g + hg * GH;
  // the sequence's row of the table: its number in the batch, or what `seq_rows` says (a table with a row per cache slot)
  const int* bt = block_table + (long)(seq_rows ? __builtin_amdgcn_readfirstlane(seq_rows[b]) : b) * table_stride;
  // the block's range of chunks, and the wave's own inside it
  const int blk_first = before + qb * 64, blk_last = before + min(qb * 64 + 63, q_len - 1);
  const int blk_lo = (window > 0 && blk_first + 1 > window) ? blk_first + 1 - window : 0;
  const int ck0 = blk_lo / 32, ck1 = blk_last / 32;
  const int qi0 = qb * 64 + wave * 16;     // first query of this wave, counted inside the step's tokens
  const bool active = qi0 < q_len;
  const bool q_ok = qi0 + j < q_len;
  const int p_mine = before + qi0 + j;                           // position of this lane's query
  const int p_last = before + min(qi0 + 15, q_len - 1);          // last position of the wave
  const int p_first = before + qi0;
  const int lo_first = (window > 0 && p_first + 1 > window) ? p_first + 1 - window : 0;
  const int lo_last = (window > 0 && p_last + 1 > window) ? p_last + 1 - window : 0;
  const int lo_mine = (window > 0 && p_mine + 1 > window) ? p_mine + 1 - window : 0;
  const int ck_first = active ? lo_first / 32 : 1, ck_last = active ? p_last / 32 : 0;

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

  // cache -> registers -> shared memory, 16 bytes a unit: a chunk's keys are 32 consecutive rows
  // of a page, its values 32 consecutive positions of each of the HS rows of the transposed page.
  // Three chunks are on their way in registers while one is worked on: a chunk's work takes a
  // fraction of a trip to memory.
  constexpr int AHEAD = 3;
  bf16x8 rk[AHEAD][NU], rv[AHEAD][NU];
  auto fetch = [&](int ck, bf16x8 (&fk)[NU], bf16x8 (&fv)[NU]) {
    const int key0 = ck * 32;
    const long page = __builtin_amdgcn_readfirstlane(bt[key0 / page_size]);
    const int po = key0 % page_size;
    // (inside a page both lie in tiles, gl3_k_offset and gl3_v_offset: the chunk's keys are still
    // 32 * HS consecutive elements, its values 512 consecutive elements for every 16 dims)
    const bf16_t* kb = k_cache + ((page * n_kv + c) * page_size + po) * HS;
    const bf16_t* vb = v_cache + (page * n_kv + c) * (long)page_size * HS + (long)(po / 8) * 128;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int u = tid + 256 * i;
      if (UNITS % 256 == 0 || u < UNITS) {
        fk[i] = *(const bf16x8*)(kb + u * 8);
        fv[i] = *(const bf16x8*)(vb + (long)(u >> 6) * page_size * 16 + (u & 63) * 8);
      }
    }
  };
  auto stage = [&](int buf, const bf16x8 (&fk)[NU], const bf16x8 (&fv)[NU]) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int u = tid + 256 * i;
      if (UNITS % 256 == 0 || u < UNITS) {
        // unit u of the keys: tile u / (2 HS) of the two, column block (u / 16) % (HS / 8), row u % 16
        const int row = u & 15, tile = u / (2 * HS);
        *(bf16x8*)&ks[buf][8 * (row >> 2) + 4 * tile + (row & 3)][((u >> 4) % (HS / 8)) * 8] = fk[i];
        // unit u of the values: 16 dims u / 64, positions 8 * ((u % 64) / 16) .., dim u % 16 of the 16
        *(bf16x8*)&vs[buf][(u >> 6) * 16 + (u & 15)][((u >> 4) & 3) * 8] = fv[i];
      }
    }
  };

  const float c2 = scale * 1.4426950408889634f;   // scores in units of log2
  const int krow = 8 * (j >> 2) + (j & 3);   // which key of a chunk is row j of the first score tile

  // one chunk of one head: scores, running softmax, weighted values. MASKED: some query of the
  // wave does not see some key of the chunk (the diagonal, a window's edge).
  auto head_chunk = [&](int hh, const bf16x8 (&ka)[KK], const bf16x8 (&kb2)[KK], const bf16x8 (&vt)[DT], int key0,
                        bool masked) {
    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kk], qt[hh][kk], sa, 0, 0, 0);
      sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb2[kk], qt[hh][kk], sb, 0, 0, 0);
    }
    float s[8];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      s[v] = sa[v];
      s[4 + v] = sb[v];
    }
    if (masked) {                               // (the same for the whole wave: a branch around the tests, one body)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int k1 = key0 + 8 * qd + v, k2 = k1 + 4;
        s[v] = (k1 >= lo_mine && k1 <= p_mine) ? s[v] : -INFINITY;
        s[4 + v] = (k2 >= lo_mine && k2 <= p_mine) ? s[4 + v] : -INFINITY;
      }
    }
    float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
    mx = max_over_quarters(mx);
    mx *= c2;                                   // c2 > 0: the greatest score stays the greatest
    const float m_new = fmaxf(m_run[hh], mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run[hh] - m_use);
    float ps = 0.f;
    bf16x8 pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float p = __builtin_amdgcn_exp2f(fmaf(s[e], c2, -m_use));
      ps += p;
      pb[e] = static_cast<bf16_t>(p);
    }
    l_run[hh] = l_run[hh] * alpha + ps;
    m_run[hh] = m_new;
    if (!__all(alpha == 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[hh][dt] *= alpha;
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[dt], pb, o[hh][dt], 0, 0, 0);
  };

#pragma unroll
  for (int r = 0; r < AHEAD; ++r)
    if (ck0 + r <= ck1) fetch(ck0 + r, rk[r], rv[r]);
  stage(0, rk[0], rv[0]);
  __syncthreads();
  int buf = 0;
  for (int base = ck0; base <= ck1; base += AHEAD) {
#pragma unroll
    for (int r = 0; r < AHEAD; ++r) {
      const int ck = base + r;
      if (ck > ck1) break;
      const int key0 = ck * 32;
      // the registers of this chunk are free (it lies in shared memory): ask for the chunk three further;
      fetch(min(ck + AHEAD, ck1), rk[r], rv[r]);   // unconditional (the last chunk again at the end): a branch
                                                   // around the loads makes the compiler wait for all of them at once
      if (ck >= ck_first && ck <= ck_last) {
        bf16x8 ka[KK], kb2[KK], vt[DT];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          ka[kk] = *(const bf16x8*)&ks[buf][krow][kk * 32 + 8 * qd];
          kb2[kk] = *(const bf16x8*)&ks[buf][krow + 4][kk * 32 + 8 * qd];
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vt[dt] = *(const bf16x8*)&vs[buf][dt * 16 + j][8 * qd];
        // every query of the wave sees the whole chunk: no mask (the same for the whole wave)
        const bool masked = !(key0 + 31 <= p_first && key0 >= lo_last);
#pragma unroll
        for (int hh = 0; hh < GH; ++hh) head_chunk(hh, ka, kb2, vt, key0, masked);
      }
      if (ck < ck1) stage(buf ^ 1, rk[(r + 1) % AHEAD], rv[(r + 1) % AHEAD]);
      __syncthreads();
      buf ^= 1;
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

// The same attention with 32 queries of one head to a wave (128 to a block) on the 32x32x16 instruction, for
// steps that bring enough queries to fill such blocks: a wave reads the chunk's keys and values out
// of shared memory once for twice as many queries, and a block brings a chunk from the cache once
// for twice as many, which is what bounds the kernel above. Tiles as there, transposed:
//   S^T[key, query]  = K[key, :] . Q[query, :]^T     one 32 x 32 tile per chunk of 32 keys
//   O^T[dim, query] += V^T[dim, key] . P^T[key, query]
// A lane holds, of the score tile, query lane % 32 and the rows 8a + 4h + b (h = lane / 32, register
// 4a + b); row r of the tile is made key 16*(a/2) + 8h + 4*(a%2) + b of the chunk by the order in
// which the key rows are read, so that registers 0..7 hold the keys 8h..8h+7 of the chunk's first
// half and registers 8..15 those of its second half: the order in which the second product takes
// its 16 keys a step.
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int HS, int CK, int AHEAD, int OCC>
__global__ __launch_bounds__(256, OCC) void attention_prefill_wide_kernel(
    const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ cu_seqlens, const int* __restrict__ kv_before, const int* __restrict__ block_table,
    const int* __restrict__ seq_rows, int table_stride, bf16_t* __restrict__ out, long out_stride, int n_heads, int n_kv, int page_size, int window,
    float scale, int q_blocks) {
  constexpr int KS = HS / 16;             // steps of the score product
  constexpr int DT = HS / 32;             // tiles of 32 dims of the output
  constexpr int NT = CK / 32;             // score tiles of a chunk of CK keys
  constexpr int KROW = HS + 8;
  constexpr int VROW = CK + 8;
  constexpr int VU = CK / 8;              // 16-byte units of a row of the transposed value chunk
  constexpr int UNITS = HS * CK / 8;      // 16-byte units of a chunk of keys (and of values)
  constexpr int NU = (UNITS + 255) / 256;
  constexpr int QB = 128;                 // queries of a block
  __shared__ __attribute__((aligned(16))) bf16_t ks[2][CK][KROW];
  __shared__ __attribute__((aligned(16))) bf16_t vs[2][HS][VROW];
  const int g = n_heads / n_kv;
  const int qb = q_blocks - 1 - blockIdx.z;      // the longest query blocks of all heads and sequences first
  const int b = blockIdx.y;
  const int head = blockIdx.x, c = head / g;   // one query head to a block
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int n = lane & 31, h = lane >> 5;
  const int tok0 = __builtin_amdgcn_readfirstlane(cu_seqlens[b]);
  const int q_len = __builtin_amdgcn_readfirstlane(cu_seqlens[b + 1]) - tok0;
  if (qb * QB >= q_len) return;            // the whole block: no barrier has been passed yet
  const int before = __builtin_amdgcn_readfirstlane(kv_before[b]);
  // the sequence's row of the table: its number in the batch, or what `seq_rows` says (a table with a row per cache slot)
  const int* bt = block_table + (long)(seq_rows ? __builtin_amdgcn_readfirstlane(seq_rows[b]) : b) * table_stride;
  const int blk_first = before + qb * QB, blk_last = before + min(qb * QB + QB - 1, q_len - 1);
  const int blk_lo = (window > 0 && blk_first + 1 > window) ? blk_first + 1 - window : 0;
  const int ck0 = blk_lo / CK, ck1 = blk_last / CK;
  const int qi0 = qb * QB + wave * 32;
  const bool active = qi0 < q_len;
  const bool q_ok = qi0 + n < q_len;
  const int p_mine = before + qi0 + n;
  const int p_last = before + min(qi0 + 31, q_len - 1);
  const int p_first = before + qi0;
  const int lo_first = (window > 0 && p_first + 1 > window) ? p_first + 1 - window : 0;
  const int lo_last = (window > 0 && p_last + 1 > window) ? p_last + 1 - window : 0;
  const int lo_mine = (window > 0 && p_mine + 1 > window) ? p_mine + 1 - window : 0;
  const int ck_first = active ? lo_first / CK : 1, ck_last = active ? p_last / CK : 0;

  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 qt[KS];
#pragma unroll
  for (int kk = 0; kk < KS; ++kk)
    qt[kk] = q_ok ? *(const bf16x8*)(q + (long)(tok0 + qi0 + n) * q_stride + (long)head * HS + kk * 16 + 8 * h) : zero8;

  float m_run = -INFINITY, l_run = 0.f;
  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[dt][v] = 0.f;

  bf16x8 rk[AHEAD][NU], rv[AHEAD][NU];
  auto fetch = [&](int ck, bf16x8 (&fk)[NU], bf16x8 (&fv)[NU]) {
    const int key0 = ck * CK;
    const long page = __builtin_amdgcn_readfirstlane(bt[key0 / page_size]);
    const int po = key0 % page_size;
    // (inside a page both lie in tiles, gl3_k_offset and gl3_v_offset: the chunk's keys are still
    // CK * HS consecutive elements, its values CK * 16 consecutive elements for every 16 dims)
    const bf16_t* kb = k_cache + ((page * n_kv + c) * page_size + po) * HS;
    const bf16_t* vb = v_cache + (page * n_kv + c) * (long)page_size * HS + (long)(po / 8) * 128;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int u = tid + 256 * i;
      if (UNITS % 256 == 0 || u < UNITS) {
        fk[i] = *(const bf16x8*)(kb + u * 8);
        fv[i] = *(const bf16x8*)(vb + (long)(u / (2 * CK)) * page_size * 16 + (u % (2 * CK)) * 8);
      }
    }
  };
  auto stage = [&](int buf, const bf16x8 (&fk)[NU], const bf16x8 (&fv)[NU]) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int u = tid + 256 * i;
      if (UNITS % 256 == 0 || u < UNITS) {
        // unit u of the keys: 32 keys u / (4 HS), of their two tiles (u / (2 HS)) % 2, column block
        // (u / 16) % (HS / 8), row u % 16
        const int row = u & 15, tile = (u / (2 * HS)) & 1, group = u / (4 * HS);
        *(bf16x8*)&ks[buf][32 * group + 8 * (row >> 2) + 4 * tile + (row & 3)][((u >> 4) % (HS / 8)) * 8] = fk[i];
        // unit u of the values: 16 dims u / (2 CK), positions 8 * ((u % (2 CK)) / 16) .., dim u % 16 of the 16
        *(bf16x8*)&vs[buf][(u / (2 * CK)) * 16 + (u & 15)][((u % (2 * CK)) >> 4) * 8] = fv[i];
      }
    }
  };

  const float c2 = scale * 1.4426950408889634f;   // scores in units of log2
  // which key of a chunk is row n of the score tile
  const int krow = 16 * (n >> 4) + 8 * ((n >> 2) & 1) + 4 * ((n >> 3) & 1) + (n & 3);

  // One chunk: scores, running softmax, weighted values. The operands are read from shared memory
  // where they are used, no more than four ahead of their products (the scheduler would read them
  // all first, and they do not fit into the registers beside the sums). MASKED: some query of the
  // wave does not see some key of the chunk (the diagonal, a window's edge).
  auto chunk = [&](int buf, int key0, bool masked) {
    f32x16 s[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) s[t][v] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {      // the tiles' sums do not depend on each other: the matrix cores stay busy
        const bf16x8 a = *(const bf16x8*)&ks[buf][32 * t + krow][kk * 16 + 8 * h];
        s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qt[kk], s[t], 0, 0, 0);
      }
      if (kk % 4 == 3) __builtin_amdgcn_sched_barrier(0);
    }
    if (masked) {                               // (the same for the whole wave: a branch around the tests, one body)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = key0 + 32 * t + 16 * (v >> 3) + 8 * h + (v & 7);
          s[t][v] = (key >= lo_mine && key <= p_mine) ? s[t][v] : -INFINITY;
        }
    }
    float mx = s[0][0];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[t][v]);
    {   // the other half of the keys of this query sits 32 lanes away
      auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
      mx = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    }
    mx *= c2;                                   // c2 > 0: the greatest score stays the greatest
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    float ps = 0.f;
    bf16x8 pb[NT][2];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[t][e], c2, -m_use));
        ps += p;
        pb[t][e >> 3][e & 7] = static_cast<bf16_t>(p);
      }
    l_run = l_run * alpha + ps;
    m_run = m_new;
    if (!__all(alpha == 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[dt] *= alpha;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const bf16x8 v0 = *(const bf16x8*)&vs[buf][dt * 32 + n][32 * t + 8 * h];
        const bf16x8 v1 = *(const bf16x8*)&vs[buf][dt * 32 + n][32 * t + 16 + 8 * h];
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v0, pb[t][0], o[dt], 0, 0, 0);
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, pb[t][1], o[dt], 0, 0, 0);
        if (dt % 2 == 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

#pragma unroll
  for (int r = 0; r < AHEAD; ++r) fetch(min(ck0 + r, ck1), rk[r], rv[r]);
  stage(0, rk[0], rv[0]);
  __syncthreads();
  int buf = 0;
  for (int base = ck0; base <= ck1; base += AHEAD) {
#pragma unroll
    for (int r = 0; r < AHEAD; ++r) {
      const int ck = base + r;
      if (ck > ck1) break;
      const int key0 = ck * CK;
      // the registers of this chunk are free (it lies in shared memory): ask for the chunk AHEAD further;
      // unconditional (the last chunk again at the end): a branch around the loads makes the compiler
      // wait for all of them at once
      fetch(min(ck + AHEAD, ck1), rk[r], rv[r]);
      if (ck >= ck_first && ck <= ck_last) {
        // every query of the wave sees the whole chunk: no mask (the same for the whole wave)
        chunk(buf, key0, !(key0 + CK - 1 <= p_first && key0 >= lo_last));
      }
      if (ck < ck1) stage(buf ^ 1, rk[(r + 1) % AHEAD], rv[(r + 1) % AHEAD]);
      __syncthreads();
      buf ^= 1;
    }
  }

  float l = l_run;
  l += __shfl_xor(l, 32, 64);
  if (!q_ok) return;
  const float inv = 1.0f / l;
  bf16_t* op = out + (long)(tok0 + qi0 + n) * out_stride + (long)head * HS + 4 * h;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      bf16x4 r;
#pragma unroll
      for (int v = 0; v < 4; ++v) r[v] = static_cast<bf16_t>(o[dt][4 * a + v] * inv);
      *(bf16x4*)(op + dt * 32 + 8 * a) = r;
    }
}

// Which of the two kernels a step takes, unless the caller says otherwise. Heads of 32 and 64: the one
// with 128 queries a block (chunks of 64 keys) from 33 tokens of the longest sequence on; it was the faster
// one at every length from there (192 tokens, 32 heads of 64: 7.4 against 9.8 us; 1,024: 23 against 33 us).
// Heads of 96 and 128: only where it has at least two blocks for every CU; below that the kernel of 64
// queries a block, with twice the blocks, is ahead (32 heads of 128, one sequence: 1,024 tokens 38 against
// 42 us, 1,536 tokens 59 against 65 us, 2,048 tokens 99 against 84 us).
static bool prefill_wide(int head_dim, int n_heads, int n_seqs, int max_q_len) {
  if (head_dim <= 64) return max_q_len > 32;
  return (long)n_heads * n_seqs * ((max_q_len + 127) / 128) >= 512;
}

extern "C" int gl3_attention_prefill_supports(int head_dim, int page_size) {
  return (head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128) && page_size % 32 == 0;
}

// max_q_len: the most tokens any sequence brings in this step (it sizes the grid).
// seq_rows (may be null): the row of `block_table` that holds sequence b's pages; null: row b.
// wide_from: the kernel with 128 queries a block is taken when max_q_len reaches it; <= 0: the library's choice.
extern "C" int gl3_attention_prefill(const void* q, long q_stride, const void* k_cache, const void* v_cache,
                                     const int* cu_seqlens, const int* kv_before, const int* block_table,
                                     const int* seq_rows, int table_stride, void* out, long out_stride, int n_seqs,
                                     int max_q_len, int n_heads, int n_kv, int head_dim, int page_size, int window,
                                     float scale, int wide_from, hipStream_t stream) {
  if (n_seqs == 0 || max_q_len == 0) return 0;
  GL3_REQUIRE(q && k_cache && v_cache && cu_seqlens && kv_before && block_table && out,
              "gl3_attention_prefill: null argument");
  GL3_REQUIRE(gl3_attention_prefill_supports(head_dim, page_size),
              "gl3_attention_prefill: head_dim %d / page_size %d is not built (32, 64, 96, 128; pages of a multiple of 32)",
              head_dim, page_size);
  GL3_REQUIRE(n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "gl3_attention_prefill: %d heads over %d kv heads",
              n_heads, n_kv);
  GL3_REQUIRE(scale > 0.f, "gl3_attention_prefill: the score scale %g must be positive", (double)scale);
  GL3_REQUIRE(q_stride % 8 == 0 && (uintptr_t)q % 16 == 0 && out_stride % 4 == 0 && (uintptr_t)out % 8 == 0,
              "gl3_attention_prefill: queries must be 16-byte aligned, outputs 8-byte aligned");
  const int g = n_heads / n_kv;
  // query heads per wave: as many as the registers hold with two blocks on a CU
  const bool wide = wide_from > 0 ? max_q_len >= wide_from : prefill_wide(head_dim, n_heads, n_seqs, max_q_len);
  // query heads per wave: as many as the registers hold with two blocks on a CU; one with 32 queries a wave
  const int gh = wide ? 1 : head_dim <= 32 ? 4 : head_dim <= 64 ? 2 : 1;
  const long z = (long)n_kv * ((g + gh - 1) / gh);
  const int q_blocks = wide ? (max_q_len + 127) / 128 : (max_q_len + 63) / 64;
  GL3_REQUIRE(n_seqs <= 65535 && q_blocks <= 65535, "gl3_attention_prefill: %d sequences / %d blocks of queries exceed the grid",
              n_seqs, q_blocks);
  dim3 grid((unsigned)z, n_seqs, q_blocks), block(256);
  if (wide) {
#define GOW(HS, CK, AH, OCC)                                                                                        \
  attention_prefill_wide_kernel<HS, CK, AH, OCC><<<grid, block, 0, stream>>>(                                       \
      (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, cu_seqlens, kv_before, block_table, \
      seq_rows, table_stride, (bf16_t*)out, out_stride, n_heads, n_kv, page_size, window, scale, q_blocks)
    // chunks of 64 keys (one barrier for twice the work, two score tiles whose sums do not wait for
    // each other) where the registers hold them and a page holds whole chunks
    const bool ck64 = page_size % 64 == 0;
    switch (head_dim) {
      case 32: if (ck64) GOW(32, 64, 2, 3); else GOW(32, 32, 2, 3); break;
      case 64: if (ck64) GOW(64, 64, 2, 2); else GOW(64, 32, 2, 3); break;
      case 96: GOW(96, 32, 2, 2); break;
      default: GOW(128, 32, 1, 2); break;
    }
#undef GOW
    GL3_LAUNCH_CHECK();
    return 0;
  }
#define GO(HS, GH)                                                                                                  \
  attention_prefill_kernel<HS, GH><<<grid, block, 0, stream>>>(                                                     \
      (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, cu_seqlens, kv_before, block_table, \
      seq_rows, table_stride, (bf16_t*)out, out_stride, n_heads, n_kv, page_size, window, scale, q_blocks)
  switch (head_dim) {
    case 32: GO(32, 4); break;
    case 64: GO(64, 2); break;
    case 96: GO(96, 1); break;
    default: GO(128, 1); break;
  }
#undef GO
  GL3_LAUNCH_CHECK();
  return 0;
}

// C[M,N] = A[M,K] . W[N,K]^T in bfloat16 for few rows of A (M <= 64): the products of
// a decode step, where every weight is read once and the time is the time to stream W.
//
// Matrix cores, 16x16x32 tiles: the 16 rows of a strip of W are the tile's rows, up to
// 64 tokens (MT tiles of 16) its columns, so a lane's 16-byte load from W (8 consecutive
// k of one row) is the operand as the instruction wants it: W goes from memory to
// registers and nowhere else. A block is NW waves (4, 8 or 16) on one strip; the waves
// share out the k-steps so that a strip's whole row range is in flight at once, and the
// NW partial tiles are summed through shared memory in wave order: the result has one
// fixed order of summation. No block ever waits for another: on this chip a block that
// waits for another block's stores has to push them through the per-XCD second-level
// caches, which costs more than the product itself. Where K is cut across blocks (the
// wide kernel) each slice's sums are stored apart and the next kernel adds them up.
// Lanes whose token row does not exist ask for nothing: a CU draws a bounded number of
// bytes a second through its first-level cache, whatever they are.
//
// A decode step is a chain of small kernels, each of which costs a few microseconds
// before it does any work, so what would be kernels of their own is folded into the
// products' ends:
//  * XNORM: the product is that of an RMSNorm (J/inference/InferenceCore.java:47-56). Its rows
//    arrive as bfloat16(weight * x), written by the kernel that completed the row of x (below),
//    and the row's 1/rms, which is a factor of the whole row, is applied to the sums at the end.
//    The sum of squares of a row arrives as partial sums (one per strip of the row's producer),
//    added up here in a fixed order.
//  * SSQ: the add epilogue also writes those partial sums of squares of the rows it completes,
//    and bfloat16(next norm's weight * x) of its columns, for the product that follows the norm.
//  * SK_QKV: the rows of W are [q heads | k heads | v heads]; the end rotates q and k by
//    the token's position and writes q to its buffer, k and v into the paged cache
//    (J/inference/InferenceCore.java:83-101). For half-split pairing a strip is made of 8
//    rows and the 8 rows half a head further, so both elements of a pair are in one tile.
// Other epilogues as in gemm_generic.hip: store, add into a float matrix, gated.
//
// Three kernels share the strip's end. The streaming one reloads its share of A for every
// strip and takes any K (with strips of 16 rows of W, or of 8 where 16 leave CUs idle). The
// resident one is for K up to 32*NW*KS: a wave keeps the A operands of its own k-steps in
// registers and the block walks over several strips with them, asking for the next strip's
// rows of W before it finishes the current strip; then the first-level cache carries W and
// nothing else, which is what limits the streaming kernel when the same A is read for every
// strip. The wide one, for 17 to 64 rows, takes several strips at once (see there).
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

enum { SK_STORE = 0, SK_ADD = 1, SK_GATED = 2, SK_QKV = 3 };

struct SkNorm {
  const float* ssq;       // [n_partials][64] partial sums of squares of the rows of x
  int n_partials;
  float eps;
  const int* rows;        // may be null: row m of the product reads row rows[m] of A
};

// What the end of a product applies or leaves besides its epilogue's own rule. For the norm that
// follows an add epilogue: its weight, and where bfloat16(weight * x) goes. For any epilogue but
// the rotation's: a bias per output column, added to the sums first (gated: the gate's biases,
// then the up's), and the activation of the gated epilogue (GL3_ACT_*).
struct SkNext {
  const float* weight;    // [N] float; null: nothing is written
  bf16_t* xg;             // [M][ld]
  long ld;
  const float* bias;      // [N] (gated: [2N]) float; null: none
  int act;
  int pack_out;           // (store and gated epilogues, at most 8 rows) the rows go out in the packed tiles' order, see sk_packed_offset
};

// Where element k of row m (< 8) of a step lies when the step's rows are kept in the order in which the
// products of at most 8 rows with packed tiles read them: [step of 64 k][lane 16 q + r][8 elements], lane
// (r, q) holding row r % 8 at k = 32 (r / 8) + 8 q. Such a product then reads 1 KB of consecutive memory
// per instruction, where rows one after the other put every lane on a line of its own; with a long K
// (the down projection) every block reads as many bytes of the step's rows as of its weights.
__device__ __forceinline__ long sk_packed_offset(int m, int k) {
  return ((long)(((k >> 6) << 6) + (((k >> 3) & 3) << 4) + (((k >> 5) & 1) << 3) + m) << 3) + (k & 7);
}

struct SkRope {
  const int* positions;
  const int* seq_of_token;
  const int* block_table;
  int table_stride;
  const float* cos_tab;   // null: no rotation
  const float* sin_tab;
  bf16_t* k_cache;
  bf16_t* v_cache;
  int n_heads, n_kv, head_dim, adjacent, page_size;
};

// Which row of W is row r of a strip's tile, and for SK_QKV which head the strip belongs to.
// A strip is ROWS rows of W: 16, or 8 (then rows 8..15 of the tile repeat rows 0..7 and are not
// written: half a tile is wasted for twice as many blocks where 16-row strips leave CUs idle).
template <int EPI, int ROWS = 16>
__device__ __forceinline__ int sk_strip_row(int strip, int r, int N, const SkRope& rp, int& hd, int& sub, bool& rotated) {
  int wr = min(strip * ROWS + (r % ROWS), N - 1);
  hd = 0; sub = 0; rotated = false;
  if (EPI == SK_QKV) {
    const int per_head = rp.head_dim / 16;
    hd = strip / per_head;
    sub = strip % per_head;
    rotated = rp.cos_tab != nullptr && hd < rp.n_heads + rp.n_kv;
    if (rotated && !rp.adjacent)
      wr = hd * rp.head_dim + 8 * sub + (r < 8 ? r : rp.head_dim / 2 + r - 8);
  }
  return wr;
}

template <bool XNORM>
__device__ __forceinline__ const void* sk_x_row(const void* Av, long lda, int m, const SkNorm& nrm) {
  if (XNORM && nrm.rows) m = nrm.rows[m];
  return (const bf16_t*)Av + (long)m * lda;
}

// A operands of one k-step for MT token tiles: elements k .. k+7 of each tile's row.
template <int MT, bool XNORM>
__device__ __forceinline__ void sk_load_x(bf16x8 (&xf)[MT], const void* const (&xrow)[MT], int k, bool ok,
                                          const SkNorm& nrm) {
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
    xf[mt] = (ok && xrow[mt] != nullptr) ? *(const bf16x8*)((const bf16_t*)xrow[mt] + k) : zero;
}

// Partial sums of squares of the rows: wave w adds the partials w, w+NW, ... of row `lane`.
template <int NW>
__device__ __forceinline__ void sk_ssq_partials(float (*sm_ssq)[64], int M, const SkNorm& nrm) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float sp = 0.f;
  if (lane < M) {
    const int row = nrm.rows ? nrm.rows[lane] : lane;   // the partial sums are stored by row of A
    for (int p0 = wave; p0 < nrm.n_partials; p0 += NW * 16) {
      float v[16];   // sixteen loads in flight, then added in order
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int p = p0 + NW * i;
        v[i] = p < nrm.n_partials ? nrm.ssq[(long)p * 64 + row] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) sp += v[i];
    }
  }
  sm_ssq[wave][lane] = sp;
}

// What a strip's epilogue reads besides the sums, asked for before the main loop so that the
// epilogue does not wait for memory again: the residual values it adds to (add epilogue), the
// token's position, its cache page and the rotation's cos and sin (SK_QKV). Wave `mt` finishes
// token tile `mt`; a lane holds 4 columns of one token.
struct SkPre {
  f32x4 prev;
  f32x4 bias, bias_up;   // the biases of this lane's columns (zero without a bias)
  f32x4 next_w;     // the next norm's weight at this lane's columns
  f32x4 co, si;
  int pos;
  int page;
};

// GIVEN (SK_QKV): the caller has asked for the token's position and its row of the block table already
// (`pos`, `table_row`), so that what depends on them can be asked for without another wait.
template <int MT, int EPI, typename TC, int ROWS = 16, bool GIVEN = false>
__device__ __forceinline__ SkPre sk_preload(const TC* __restrict__ C, int M, int N, long ldc, int strip, int hd, int sub,
                                            bool rotated, const SkRope& rp, const SkNext& nx = SkNext{}, int pos = 0,
                                            int table_row = 0) {
  SkPre p;
  p.prev = p.bias = p.bias_up = p.next_w = p.co = p.si = f32x4{0.f, 0.f, 0.f, 0.f};
  p.pos = 0; p.page = 0;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int m = wave * 16 + r;
  if (wave >= MT || m >= M || 4 * q >= ROWS) return p;
  if (EPI != SK_QKV && nx.bias) {
    const int n = strip * ROWS + 4 * q;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      if (n + c < N) {
        p.bias[c] = nx.bias[n + c];
        if (EPI == SK_GATED) p.bias_up[c] = nx.bias[N + n + c];
      }
  }
  if (EPI == SK_ADD) {
    const int n = strip * ROWS + 4 * q;
    const TC* cp = C + (long)m * ldc + n;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      if (n + c < N) {
        p.prev[c] = to_f32<TC>(cp[c]);
        if (nx.weight) p.next_w[c] = nx.weight[n + c];
      }
  }
  if (EPI == SK_QKV) {
    p.pos = GIVEN ? pos : rp.positions[m];
    if (hd >= rp.n_heads)
      p.page = rp.block_table[(long)(GIVEN ? table_row : rp.seq_of_token[m]) * rp.table_stride + p.pos / rp.page_size];
    if (rotated) {
      const int half = rp.head_dim / 2;
      if (rp.adjacent) {
        const int jj = (16 * sub + 4 * q) / 2;
        p.co[0] = rp.cos_tab[(long)p.pos * half + jj];     p.si[0] = rp.sin_tab[(long)p.pos * half + jj];
        p.co[1] = rp.cos_tab[(long)p.pos * half + jj + 1]; p.si[1] = rp.sin_tab[(long)p.pos * half + jj + 1];
      } else {
        const int jj = 8 * sub + 4 * (q & 1);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          p.co[c] = rp.cos_tab[(long)p.pos * half + jj + c];
          p.si[c] = rp.sin_tab[(long)p.pos * half + jj + c];
        }
      }
    }
  }
  return p;
}

// The end of a strip: the waves' partial tiles are summed in wave order by the wave that owns
// the tile, then the epilogue runs. `sub`, `hd`, `rotated` describe the strip for SK_QKV.
template <int MT, int NW, int EPI, typename TC, bool XNORM, bool SSQ, int ROWS = 16>
__device__ __forceinline__ void sk_finish(f32x4 (*red)[((EPI == SK_GATED) ? 2 : 1) * MT][64], float (*sm_ssq)[64],
                                          const f32x4 (&acc)[(EPI == SK_GATED) ? 2 : 1][MT], int strip, int hd, int sub,
                                          bool rotated, TC* __restrict__ C, int M, int N, int K, long ldc,
                                          const SkNorm& nrm, float* __restrict__ ssq_out, const SkRope& rp,
                                          const SkNext& nx, const SkPre& pre) {
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int n0 = strip * ROWS;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[wave][g * MT + mt][lane] = acc[g][mt];
  __syncthreads();
  for (int t = wave; t < NG * MT; t += NW) {
    f32x4 v = red[0][t][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) v += red[w][t][lane];
    red[0][t][lane] = v;   // only this thread touches red[*][t][lane] before the barrier
  }
  __syncthreads();

  // epilogue: lane holds tile rows 4q .. 4q+3 (columns of C) of token mt*16 + r
  for (int mt = wave; mt < MT; mt += NW) {
    const int m = mt * 16 + r;
    const bool m_ok = m < M;
    f32x4 v = red[0][mt][lane];
    f32x4 up = (EPI == SK_GATED) ? red[0][MT + mt][lane] : zero4;
    if (XNORM) {
      float ss = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) ss += sm_ssq[w][min(m, 63)];
      const float rms = 1.0f / sqrtf(ss / (float)K + nrm.eps);
      v *= rms;
      up *= rms;
    }
    if (EPI != SK_QKV) {
      v += pre.bias;
      up += pre.bias_up;
    }
    if (EPI == SK_GATED) {
#pragma unroll
      for (int c = 0; c < 4; ++c) v[c] = gl3_activation<true>(v[c], nx.act) * up[c];
    }
    if (EPI == SK_QKV) {
      const int hs = rp.head_dim;
      const int pos = pre.pos;
      int col = 16 * sub + 4 * q;          // first of this lane's 4 columns inside the head
      if (rotated) {
        const int half = hs / 2;
        if (rp.adjacent) {
          const float c0 = pre.co[0], s0 = pre.si[0];
          const float c1 = pre.co[1], s1 = pre.si[1];
          const f32x4 o = v;
          v[0] = o[0] * c0 - o[1] * s0;
          v[1] = o[0] * s0 + o[1] * c0;
          v[2] = o[2] * c1 - o[3] * s1;
          v[3] = o[2] * s1 + o[3] * c1;
        } else {
          // quarters 0,1 hold the first elements of 8 pairs, quarters 2,3 their partners
          const bool first = q < 2;
          const int jj = 8 * sub + 4 * (q & 1);
          col = (first ? 0 : half) + jj;
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const float other = __shfl_xor(v[c], 32, 64);
            const float co = pre.co[c], si = pre.si[c];
            v[c] = first ? v[c] * co - other * si : other * si + v[c] * co;
          }
        }
      }
      if (m_ok) {
        if (hd < rp.n_heads) {
          bf16x4 o4;
#pragma unroll
          for (int c = 0; c < 4; ++c) o4[c] = static_cast<bf16_t>(v[c]);
          *(bf16x4*)((bf16_t*)C + (long)m * ldc + (long)hd * hs + col) = o4;
        } else {
          const long page = pre.page;
          const int in_page = pos % rp.page_size;
          if (hd < rp.n_heads + rp.n_kv) {
            const int ch = hd - rp.n_heads;
            bf16x4 o4;
#pragma unroll
            for (int c = 0; c < 4; ++c) o4[c] = static_cast<bf16_t>(v[c]);
            *(bf16x4*)(rp.k_cache + (page * rp.n_kv + ch) * (long)rp.page_size * hs + gl3_k_offset(in_page, col, hs)) = o4;
          } else {
            const int ch = hd - rp.n_heads - rp.n_kv;
            bf16_t* vt = rp.v_cache + (page * rp.n_kv + ch) * (long)rp.page_size * hs + gl3_v_offset(col, in_page, rp.page_size);
#pragma unroll
            for (int c = 0; c < 4; ++c) vt[8 * c] = static_cast<bf16_t>(v[c]);   // (col % 4 == 0: the 4 dims lie in one tile)
          }
        }
      }
      continue;
    }
    const int n = n0 + 4 * q;
    TC* cp = (EPI != SK_ADD && nx.pack_out) ? C + sk_packed_offset(m & 7, n) : C + (long)m * ldc + n;
    float sq = 0.f;
    if (m_ok && 4 * q < ROWS) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (n + c < N) {
          float o = v[c];
          if (EPI == SK_ADD) o += pre.prev[c];
          cp[c] = from_f32<TC>(o);
          sq += o * o;
          if (SSQ && nx.weight) nx.xg[(long)m * nx.ld + n + c] = static_cast<bf16_t>(pre.next_w[c] * o);
        }
      }
    }
    if (SSQ) {
      sq += __shfl_xor(sq, 16, 64);
      sq += __shfl_xor(sq, 32, 64);
      if (q == 0 && m_ok) ssq_out[(long)strip * 64 + m] = sq;
    }
  }
}

// PACK (strips of 8 rows, at most 8 rows of A, one token tile): the tile's rows 8..15 are the strip's
// 8 rows again, 32 k further, and its token columns 8..15 the tokens again at those k, so that one
// instruction covers 64 k of the strip, every lane loads (a row of W and a row of A are read in
// whole 128-byte lines) and nothing of the tile is idle. Of the 16 x 16 sums the two diagonal
// 8 x 8 blocks are the product's two halves, added at the end; the other two are dropped.
template <int MT, int NW, int EPI, typename TC, bool XNORM, bool SSQ, int ROWS = 16, bool PACK = false>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const void* __restrict__ Av, const bf16_t* __restrict__ W,
                                                              TC* __restrict__ C, int M, int N, int K, long lda,
                                                              long ldw, long ldc, SkNorm nrm, float* __restrict__ ssq_out,
                                                              SkNext nx, SkRope rp, const bf16_t* __restrict__ Wt8, int a_packed) {
  static_assert(!PACK || (ROWS == 8 && MT == 1 && EPI != SK_GATED && EPI != SK_QKV && !XNORM), "packed strips: 8 rows, one tile");
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  constexpr int UNROLL = 8;
  __shared__ f32x4 red[NW][NG * MT][64];
  __shared__ float sm_ssq[XNORM ? NW : 1][64];
  const int strip = blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  int hd, sub;
  bool rotated;
  const int wr = sk_strip_row<EPI, ROWS>(strip, r, N, rp, hd, sub, rotated);
  const int koff = PACK ? 32 * (r >> 3) + q * 8 : q * 8;   // the lane's place inside a k-step
  const bf16_t* wrow = W + (long)wr * ldw + koff;
  const bf16_t* urow = wrow + (long)N * ldw;  // up rows (gated only)
  const void* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {   // null for rows that do not exist: their lanes ask for nothing
    const int m = PACK ? (r & 7) : mt * 16 + r;
    xrow[mt] = m < M ? sk_x_row<XNORM>(Av, lda, m, nrm) : nullptr;
  }
  if (XNORM) sk_ssq_partials<NW>(sm_ssq, M, nrm);
  const SkPre pre = sk_preload<MT, EPI, TC, ROWS>(C, M, N, ldc, strip, hd, sub, rotated, rp, nx);

  const int steps = (K + 31) / 32;   // k-steps of 32
  f32x4 acc[NG][MT];
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[g][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  if (PACK) {
    // a wave takes steps of 64 k: step wave, wave + NW, ...
    // (Wt8, may be null: W as [strip of 8 rows][step of 64 k][lane][8], the packed tile's own order, k padded
    // with zeros to whole steps: a load is then 1 KB of consecutive memory)
    const int steps64 = (K + 63) / 64;
    const bf16_t* wbase = Wt8 ? Wt8 + ((long)strip * steps64 * 64 + lane) * 8 : wrow;
    const long w_step = Wt8 ? 512 : 64;
    for (int p0 = wave; p0 * 64 < K; p0 += NW * UNROLL) {
      bf16x8 wf[UNROLL], xf[UNROLL][MT];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int p = p0 + NW * u, k = p * 64;
        const bool ok = k + koff < K;   // K is a multiple of 8: a lane's 8 elements are all in or all out
        wf[u] = (Wt8 ? p < steps64 : ok) ? *(const bf16x8*)(wbase + p * w_step) : zero;
        if (a_packed)   // the rows in the packed tiles' order (sk_packed_offset): this lane's 16 bytes of step p
          xf[u][0] = (ok && xrow[0] != nullptr) ? *(const bf16x8*)((const bf16_t*)Av + ((long)p * 64 + lane) * 8) : zero;
        else
          sk_load_x<MT, XNORM>(xf[u], xrow, k + koff, ok, nrm);
      }
      __builtin_amdgcn_sched_barrier(0);   // all of the batch's loads are issued before the first is waited for
#pragma unroll
      for (int u = 0; u < UNROLL; ++u)
        acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u], xf[u][0], acc[0][0], 0, 0, 0);
    }
    // lane (token column j, quarter q) holds tile rows 4q .. 4q+3: the sums over the first 32 k of every
    // step lie at j < 8, q < 2, those over the second at j >= 8, q >= 2: lane + 40
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[0][0][c] += __shfl_xor(acc[0][0][c], 40, 64);
  } else {
  // a wave takes pairs of neighbouring k-steps (the two halves of one 128-byte line of a row of W):
  // pair wave, wave + NW, ...
  // (strips of 16 rows: Wt8, may be null, is W as [strip][k-step of 32][lane][8], the operands' own order,
  // k padded with zeros to whole steps; gated: the up strips follow the N / 16 gate strips)
  const bool tiled = ROWS == 16 && Wt8 != nullptr;
  const bf16_t* wbase = tiled ? Wt8 + ((long)strip * steps * 64 + lane) * 8 : wrow;
  const bf16_t* ubase = tiled ? wbase + (long)(N / 16) * steps * 512 : urow;
  const long w_step = tiled ? 512 : 32;
  for (int p0 = wave; 2 * p0 < steps; p0 += NW * (UNROLL / 2)) {
    bf16x8 wf[UNROLL], uf[UNROLL], xf[UNROLL][MT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int st = 2 * (p0 + NW * (u / 2)) + (u & 1), k = st * 32;
      const bool ok = k + q * 8 < K;   // K is a multiple of 8: a lane's 8 elements are all in or all out
      const bool w_ok = tiled ? st < steps : ok;
      wf[u] = (w_ok && r < ROWS) ? *(const bf16x8*)(wbase + st * w_step) : zero;   // rows of the tile beyond the strip stay zero
      if (EPI == SK_GATED) uf[u] = w_ok ? *(const bf16x8*)(ubase + st * w_step) : zero;
      sk_load_x<MT, XNORM>(xf[u], xrow, k + q * 8, ok, nrm);
    }
    __builtin_amdgcn_sched_barrier(0);   // all of the batch's loads are issued before the first is waited for
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        acc[0][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u], xf[u][mt], acc[0][mt], 0, 0, 0);
        if (EPI == SK_GATED) acc[1][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[u], xf[u][mt], acc[1][mt], 0, 0, 0);
      }
    }
  }
  }
  sk_finish<MT, NW, EPI, TC, XNORM, SSQ, ROWS>(red, sm_ssq, acc, strip, hd, sub, rotated, C, M, N, K, ldc, nrm, ssq_out, rp,
                                               nx, pre);
}

// The resident kernel: K <= 32 * NW * KS. `n_strips` strips are shared out over the blocks.
template <int MT, int NW, int KS, int EPI, typename TC, bool XNORM, bool SSQ>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_resident_kernel(
    const void* __restrict__ Av, const bf16_t* __restrict__ W, TC* __restrict__ C, int M, int N, int K, long lda,
    long ldw, long ldc, SkNorm nrm, float* __restrict__ ssq_out, SkNext nx, SkRope rp, int n_strips,
    const bf16_t* __restrict__ Wt) {
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  __shared__ f32x4 red[NW][NG * MT][64];
  __shared__ float sm_ssq[XNORM ? NW : 1][64];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // Where a strip's operands lie. In W itself a lane's 16 bytes of k-step s are in its row at 32 s
  // elements; every lane of a load is then on a line of its own. In the copy in the operands' own
  // order (Wt, may be null: [strip][k-step][lane][8], k padded with zeros to whole steps, the strips'
  // rows as sk_strip_row names them) a load is 1 KB of consecutive memory, which the CU's first-level
  // cache takes in less than half the time.
  const int steps_all = (K + 31) / 32;
  const long w_step = Wt ? 512 : 32;                       // elements from one k-step to the next
  const long w_up = Wt ? (long)(N / 16) * steps_all * 512 : (long)N * ldw;   // from a gate strip to its up strip
  auto strip_base = [&](int strip_, int& hd_, int& sub_, bool& rot_) {
    const int wr = sk_strip_row<EPI>(strip_, r, N, rp, hd_, sub_, rot_);
    return Wt ? Wt + ((long)strip_ * steps_all * 64 + lane) * 8 : W + (long)wr * ldw + q * 8;
  };
  auto step_ok = [&](int st) { return Wt ? st < steps_all : st * 32 + q * 8 < K; };
  // Everything the block needs first is asked for before anything is waited for, so that it all
  // arrives in one trip to memory: the first strip's rows of W, the rows' partial sums of squares,
  // and this wave's share of A (k-steps wave, wave + NW, ...).
  int strip = blockIdx.x;
  int hd, sub;
  bool rotated;
  bf16x8 wf[KS], uf[KS];
  {
    const bf16_t* wrow = strip_base(strip, hd, sub, rotated);
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const int st = wave + NW * i;
      const bool ok = step_ok(st);
      wf[i] = ok ? *(const bf16x8*)(wrow + st * w_step) : zero;
      if (EPI == SK_GATED) uf[i] = ok ? *(const bf16x8*)(wrow + w_up + st * w_step) : zero;
    }
  }
  float sq[16];
  int sq_row = 0;
  if (XNORM) {
    sq_row = (lane < M && nrm.rows) ? nrm.rows[lane] : lane;   // the partial sums are stored by row of A
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int p = wave + NW * i;
      sq[i] = (lane < M && p < nrm.n_partials) ? nrm.ssq[(long)p * 64 + sq_row] : 0.f;
    }
  }
  bf16x8 xf[KS][MT];
  {
    const void* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)   // null for rows that do not exist: their lanes ask for nothing
      xrow[mt] = mt * 16 + r < M ? sk_x_row<XNORM>(Av, lda, mt * 16 + r, nrm) : nullptr;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const int k = (wave + NW * i) * 32 + q * 8;
      const bool ok = k < K;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        xf[i][mt] = (ok && xrow[mt] != nullptr) ? *(const bf16x8*)((const bf16_t*)xrow[mt] + k) : zero;
    }
  }
  bool first_strip = true;
  while (strip < n_strips) {
    // ask for the next strip's rows before this strip's are used
    const int next = strip + gridDim.x;
    bf16x8 wn[KS], un[KS];
    int hd_n = 0, sub_n = 0;
    bool rot_n = false;
    if (next < n_strips) {
      const bf16_t* wrow = strip_base(next, hd_n, sub_n, rot_n);
#pragma unroll
      for (int i = 0; i < KS; ++i) {
        const int st = wave + NW * i;
        const bool ok = step_ok(st);
        wn[i] = ok ? *(const bf16x8*)(wrow + st * w_step) : zero;
        if (EPI == SK_GATED) un[i] = ok ? *(const bf16x8*)(wrow + w_up + st * w_step) : zero;
      }
    }
    const SkPre pre = sk_preload<MT, EPI, TC>(C, M, N, ldc, strip, hd, sub, rotated, rp, nx);
    __builtin_amdgcn_sched_barrier(0);   // the next strip's loads are on their way before this strip's are used
    f32x4 acc[NG][MT];
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[g][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < KS; ++i) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        acc[0][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i], xf[i][mt], acc[0][mt], 0, 0, 0);
        if (EPI == SK_GATED) acc[1][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[i], xf[i][mt], acc[1][mt], 0, 0, 0);
      }
    }
    if (XNORM && first_strip) {
      // (waited for only now: the second strip's rows of W were asked for in the same trip)
      float sp = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) sp += sq[i];
      for (int p0 = wave + NW * 16; p0 < nrm.n_partials; p0 += NW * 16) {   // further partial sums, sixteen at a time
        float more[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int p = p0 + NW * i;
          more[i] = (lane < M && p < nrm.n_partials) ? nrm.ssq[(long)p * 64 + sq_row] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) sp += more[i];
      }
      sm_ssq[wave][lane] = sp;
      first_strip = false;
    }
    sk_finish<MT, NW, EPI, TC, XNORM, SSQ>(red, sm_ssq, acc, strip, hd, sub, rotated, C, M, N, K, ldc, nrm, ssq_out, rp,
                                           nx, pre);
    if (next >= n_strips) break;
    __syncthreads();   // the partial tiles in shared memory are free again
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      wf[i] = wn[i];
      if (EPI == SK_GATED) uf[i] = un[i];
    }
    strip = next; hd = hd_n; sub = sub_n; rotated = rot_n;
  }
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bf16x8 sk_buffer_load(__amdgpu_buffer_rsrc_t buf, unsigned byte_offset) {
  return __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(buf, byte_offset, 0, 0));
}

// The wide kernel, for steps of two to four token tiles: there a strip's share of A is as
// large as the strip of W itself (or larger), and reading it again for every strip is what takes the time.
// A block works on NS strips at once (NS pairs of gate and up strips for the gated epilogue), so
// that A is read once for all of them, and on one slice of K only (blockIdx.y), so that the
// chip still has blocks enough. With more than one slice the epilogue is a plain store of the
// slice's sums into slice `blockIdx.y` of a float buffer [slices][M][ldc]: whoever reads the
// result next adds the slices up in order, no block waits for another.
//
// How the operands arrive. A load in the matrix operand's own layout (lane r, q: row r, 16 bytes
// at q) touches 16 rows with 64 bytes each; a CU's first-level cache takes one such lane a clock,
// 37 GB/s a CU, whatever the second-level cache could deliver (measured; the same bytes asked for
// as 8 rows of whole 128-byte lines come at 110 GB/s). With 64 rows of A a block asks for four
// bytes of A per byte of W, all from the second-level cache, and that rate is the kernel's time.
// So a wave loads its share of both operands as whole lines (lane l: row l/8, 16 bytes at l%8;
// two loads cover a tile of 16 rows over 64 k, two k-steps), writes them into its own piece of
// shared memory and reads the tile back in the operand's layout. Inside a tile row i lies at line
// i (i < 8) or 8 + (i+1)%8, and its 16-byte piece c at (c xor i%8): then neither the writes (8 lanes
// a line) nor the reads (16 rows of one piece) meet in a bank. The piece of shared memory is the
// wave's own, so only the wave's own order matters: a fence of wavefront scope keeps the compiler
// from moving the reads over the writes, the hardware works a wave's accesses in order.
//
// XNORM (one slice of K): the product is that of an RMSNorm, as in the other kernels: A holds
// bfloat16(weight * x) and the rows' 1/rms, from the partial sums of squares, is applied to the sums.
template <int MT, int NS, int NW, int EPI, typename TC, bool XNORM>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_wide_kernel(const bf16_t* __restrict__ A,
                                                                   const bf16_t* __restrict__ W, TC* __restrict__ C,
                                                                   int M, int N, int K, long lda, long ldw, long ldc,
                                                                   long slice_stride, int pairs_per_slice, SkRope rp,
                                                                   SkNext nx, SkNorm nrm) {
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  constexpr int NWT = NS * NG;        // tiles of W a pair of k-steps
  constexpr int NT = NWT + MT;        // tiles a wave stages for a pair of k-steps: 16 rows x 128 bytes each
  constexpr int STAGE = NW * NT * 2048, RED = NW * NG * MT * 1024;
  __shared__ __attribute__((aligned(16))) char smem[STAGE > RED ? STAGE : RED];
  __shared__ float sm_ssq[XNORM ? NW : 1][64];
  f32x4 (*red)[NG * MT][64] = (f32x4 (*)[NG * MT][64])smem;   // the partial tiles, once the staging is over
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int l8 = lane >> 3, c8 = lane & 7;
  const int n_strips = (N + 15) / 16;
  const int strip0 = blockIdx.x * NS;
  char* stage = smem + wave * (NT * 2048);
  // where this lane's loads go inside a tile (rows l8 and 8 + l8) and where its operands lie (k-steps 0, 1)
  const int put0 = l8 * 128 + ((c8 ^ l8) * 16);
  const int put1 = (8 + ((l8 + 1) & 7)) * 128 + ((c8 ^ l8) * 16);
  const int line = r < 8 ? r : 8 + ((r + 1) & 7);
  const int get0 = line * 128 + ((q ^ (r & 7)) * 16);
  const int get1 = line * 128 + (((4 + q) ^ (r & 7)) * 16);

  // Both operands are read through buffer descriptors: a lane whose row or k does not exist gives
  // an offset beyond the buffer and gets zeros without a branch around the load, so every wave issues
  // the same loads in the same order and can wait for exactly the ones it needs.
  const __amdgpu_buffer_rsrc_t w_buf =
      __builtin_amdgcn_make_buffer_rsrc((void*)W, 0, (int)((((long)NG * N - 1) * ldw + K) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t a_buf =
      __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (int)((((long)M - 1) * lda + K) * 2), 0x00020000);
  constexpr unsigned NOWHERE = 0x80000000u;   // beyond any buffer the entry point lets in
  int hd[NS], sub[NS];
  bool rotated[NS];
  unsigned wo[NWT][2];   // byte offsets of this lane's lines at k = 0
#pragma unroll
  for (int g = 0; g < NS; ++g)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int wr = sk_strip_row<EPI>(min(strip0 + g, n_strips - 1), 8 * j + l8, N, rp, hd[g], sub[g], rotated[g]);
#pragma unroll
      for (int h = 0; h < NG; ++h) wo[g * NG + h][j] = (unsigned)((((long)wr + (long)h * N) * ldw + c8 * 8) * 2);
    }
  unsigned xo[MT][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int m = mt * 16 + 8 * j + l8;
      xo[mt][j] = m < M ? (unsigned)(((long)m * lda + c8 * 8) * 2) : NOWHERE;
    }

  TC* out = C + (long)blockIdx.y * slice_stride;
  // The rotation's end needs the token's position, and through it a page number and cos and sin:
  // two trips to memory one after the other. The position is asked for before the first lines of the
  // product, what hangs on it right after them, so that both trips run beside the product's first.
  int tok_pos = 0, tok_row = 0;
  if (EPI == SK_QKV) {
    const int m = min(min(wave, MT - 1) * 16 + r, M - 1);
    tok_pos = rp.positions[m];
    tok_row = rp.seq_of_token[m];
  }

  const int pairs = (K + 63) / 64;
  const int p_begin = blockIdx.y * pairs_per_slice;
  const int p_end = min(pairs, p_begin + pairs_per_slice);
  f32x4 acc[NS][NG][MT];
#pragma unroll
  for (int g = 0; g < NS; ++g)
#pragma unroll
    for (int h = 0; h < NG; ++h)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[g][h][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // The lines of one pair of k-steps are on their way while the pair before is worked on. (Asking for
  // W two pairs ahead, with the waits counted so that the later pair stays on its way, gained 3 % where
  // the registers allowed it and spilled where they did not.)
  // A wave's pairs are wave, wave + NW, ...; blocks start at different ones, so that at any time the
  // chip asks for all parts of the rows of W and not for the same quarter of every row.
  const int n_it = (p_end - p_begin + NW - 1) / NW;
  const int rot = n_it > 0 ? (int)(blockIdx.x % (unsigned)n_it) : 0;
  auto pair_at = [&](int i) {   // (i >= n_it: past the end)
    const int j = i + rot;
    return i < n_it ? p_begin + wave + NW * (j < n_it ? j : j - n_it) : p_end;
  };
  bf16x8 held[NT][2];
  auto ask = [&](int p) {
    const unsigned k2 = (p < p_end && p * 64 + c8 * 8 < K) ? (unsigned)p * 128u : NOWHERE;   // (K is a multiple of 8)
#pragma unroll
    for (int t = 0; t < NWT; ++t)
#pragma unroll
      for (int j = 0; j < 2; ++j) held[t][j] = sk_buffer_load(w_buf, wo[t][j] + k2);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        held[NWT + mt][j] = sk_buffer_load(a_buf, ((xo[mt][j] | k2) & NOWHERE) ? NOWHERE : xo[mt][j] + k2);
  };
  ask(pair_at(0));
  SkPre pre[NS];
#pragma unroll
  for (int g = 0; g < NS; ++g)
    pre[g] = sk_preload<MT, EPI, TC, 16, EPI == SK_QKV>(out, M, N, ldc, min(strip0 + g, n_strips - 1), hd[g], sub[g],
                                                         rotated[g], rp, nx, tok_pos, tok_row);
  if (XNORM) sk_ssq_partials<NW>(sm_ssq, M, nrm);   // (read after the barrier before the first strip's end)
  for (int i = 0; i < n_it; ++i) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      *(bf16x8*)(stage + t * 2048 + put0) = held[t][0];
      *(bf16x8*)(stage + t * 2048 + put1) = held[t][1];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    ask(pair_at(i + 1));
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int get = s ? get1 : get0;
      bf16x8 xf[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xf[mt] = *(const bf16x8*)(stage + (NWT + mt) * 2048 + get);
#pragma unroll
      for (int g = 0; g < NS; ++g)
#pragma unroll
        for (int h = 0; h < NG; ++h) {
          const bf16x8 wf = *(const bf16x8*)(stage + (g * NG + h) * 2048 + get);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[g][h][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf[mt], acc[g][h][mt], 0, 0, 0);
        }
    }
    // the next pair's lines are written only after this pair's operands have been read
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
#pragma unroll
  for (int g = 0; g < NS; ++g) {
    __syncthreads();   // the staged lines, then the partial tiles of the strip before, are free
    if (strip0 + g < n_strips)   // the same for all threads of the block
      sk_finish<MT, NW, EPI, TC, XNORM, false>(red, sm_ssq, acc[g], strip0 + g, hd[g], sub[g], rotated[g], out, M, N, K,
                                                ldc, nrm, nullptr, rp, nx, pre[g]);
  }
}

struct SkCall {
  const void* A; const void* W; void* C;
  int M, N, K; long lda, ldw, ldc;
  SkNorm nrm; float* ssq_out; SkRope rp;
  hipStream_t stream;
  bool resident = true;
  int strip_rows = 16;
  SkNext nx = SkNext{};
  const void* Wt = nullptr;   // W in the operands' order (the resident kernel reads it where it is given)
  const void* Wt8 = nullptr;  // W in the order of the packed tiles of strips of 8 rows
  int a_packed = 0;           // the rows of A lie in the packed tiles' order (strips of 8 rows, M <= 8 only)
};

// Blocks of the resident kernel: every strip its own block while that still leaves CUs idle, else
// two blocks per CU that walk over the strips.
static int resident_blocks(int n_strips, int nw) {
  const int most = nw == 16 ? 256 : nw == 8 ? 512 : 1024;
  return n_strips < most ? n_strips : most;
}

template <int MT, int EPI, typename TC, bool XNORM, bool SSQ>
static int launch_skinny(int nw, const SkCall& a) {
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  dim3 grid((a.N + 15) / 16);
  const int n_strips = (a.N + 15) / 16;
  const int steps = (a.K + 31) / 32;
#define RES(NW, KS)                                                                                               \
  do {                                                                                                            \
    gemm_skinny_resident_kernel<MT, NW, KS, EPI, TC, XNORM, SSQ>                                                  \
        <<<dim3(resident_blocks(n_strips, NW)), dim3(NW * 64), 0, a.stream>>>(                                    \
            a.A, (const bf16_t*)a.W, (TC*)a.C, a.M, a.N, a.K, a.lda, a.ldw, a.ldc, a.nrm, a.ssq_out, a.nx, a.rp, n_strips, \
            (const bf16_t*)a.Wt);                                                                                 \
    GL3_LAUNCH_CHECK();                                                                                           \
    return 0;                                                                                                     \
  } while (0)
  if constexpr (MT == 1 && !XNORM && (EPI == SK_STORE || EPI == SK_ADD)) {
    if (a.strip_rows == 8) {
      // strips of 8 rows: twice the blocks, each with half the rows to stream; with at most 8 rows of A
      // the tile's other half takes the next 32 k
      if (a.M <= 8)
        gemm_skinny_kernel<MT, 16, EPI, TC, XNORM, SSQ, 8, true><<<dim3((a.N + 7) / 8), dim3(16 * 64), 0, a.stream>>>(
            a.A, (const bf16_t*)a.W, (TC*)a.C, a.M, a.N, a.K, a.lda, a.ldw, a.ldc, a.nrm, a.ssq_out, a.nx, a.rp,
            (const bf16_t*)a.Wt8, a.a_packed);
      else
        gemm_skinny_kernel<MT, 16, EPI, TC, XNORM, SSQ, 8><<<dim3((a.N + 7) / 8), dim3(16 * 64), 0, a.stream>>>(
            a.A, (const bf16_t*)a.W, (TC*)a.C, a.M, a.N, a.K, a.lda, a.ldw, a.ldc, a.nrm, a.ssq_out, a.nx, a.rp,
            (const bf16_t*)nullptr, 0);
      GL3_LAUNCH_CHECK();
      return 0;
    }
  }
  if (a.resident) {
    // very many strips (the head after a prompt): four waves a block, each with four times the share
    // of K. A block walks over fewer strips, more of them are on their way on a CU at once, and four
    // partial tiles are merged per strip, not sixteen (the head at one row: 113 -> 100 us). With the
    // norm folded in (a decode step's head) the sixteen waves are the faster ones: 97 against 103 us.
    if constexpr (NG * MT == 1 && EPI != SK_QKV && !XNORM) {
      if (steps <= 64 && n_strips >= 2048) RES(4, 16);
    }
    // 16 waves a strip where their partial tiles fit, so that a strip's rows are asked for at once
    if constexpr (NG * MT <= 2) {
      if (steps <= 64) RES(16, 4);
    }
    // (more token tiles, the gated epilogue or the rotation's operands would not fit the registers with
    // this many k-steps a wave: those take the streaming kernel for a longer K)
    if constexpr (NG * MT == 1 && EPI != SK_QKV) {
      if (steps <= 128) RES(16, 8);
    }
    if constexpr (NG * MT <= 4) {
      if (steps <= 64) RES(8, 8);
    }
    if constexpr (MT == 1 && EPI != SK_GATED && EPI != SK_QKV) {
      if (steps <= 128) RES(8, 16);
    }
  }
#undef RES
#define GO(NW)                                                                                                    \
  gemm_skinny_kernel<MT, NW, EPI, TC, XNORM, SSQ><<<grid, dim3(NW * 64), 0, a.stream>>>(                          \
      a.A, (const bf16_t*)a.W, (TC*)a.C, a.M, a.N, a.K, a.lda, a.ldw, a.ldc, a.nrm, a.ssq_out, a.nx, a.rp,          \
      (const bf16_t*)a.Wt, 0)
  if constexpr (NG * MT <= 2) {
    if (nw >= 16) { GO(16); GL3_LAUNCH_CHECK(); return 0; }
  }
  if constexpr (NG * MT <= 4) {
    if (nw >= 8) { GO(8); GL3_LAUNCH_CHECK(); return 0; }
  }
  GO(4);
#undef GO
  GL3_LAUNCH_CHECK();
  return 0;
}

template <int EPI, typename TC, bool XNORM, bool SSQ>
static int pick_mt(int nw, const SkCall& a) {
  switch ((a.M + 15) / 16) {
    case 1: return launch_skinny<1, EPI, TC, XNORM, SSQ>(nw, a);
    case 2: return launch_skinny<2, EPI, TC, XNORM, SSQ>(nw, a);
    case 3: return launch_skinny<3, EPI, TC, XNORM, SSQ>(nw, a);
    default: return launch_skinny<4, EPI, TC, XNORM, SSQ>(nw, a);
  }
}

static int pick_waves(int waves, int N, int K) {
  if (waves) return waves;
  // enough waves to keep every CU's memory pipeline full, at least two k-steps each
  const long strips = (N + 15) / 16, steps = (K + 31) / 32;
  waves = 4;
  while (waves < 16 && strips * waves < 4096 && steps / (waves * 2) >= 2) waves *= 2;
  return waves;
}

static int check_common(const char* who, const void* A, const void* W, const void* C, int M, int N, int K, long lda,
                        long ldw, int waves) {
  GL3_REQUIRE(A && W && C, "%s: null operand", who);
  GL3_REQUIRE(M > 0 && M <= 64, "%s: M=%d is outside 1..64", who, M);
  GL3_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0,
              "%s: K=%d, lda=%ld, ldw=%ld must be multiples of 8", who, K, lda, ldw);
  GL3_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "%s: operands must be 16-byte aligned", who);
  GL3_REQUIRE(lda >= K && ldw >= K, "%s: leading dimensions too small", who);
  GL3_REQUIRE(waves == 0 || waves == 4 || waves == 8 || waves == 16, "%s: waves=%d", who, waves);
  return 0;
}

// `waves`: 0 lets the library choose the kernel (the resident one where K allows) and its block size;
// 4, 8 or 16 ask for the streaming kernel with that many waves per block (fewer are used when the
// partial tiles of that many waves would not fit the block's shared memory).
// ssq_out (may be null, add epilogue only, N % 16 == 0): [N/16][64] partial sums of squares of the
// completed rows.
// strip_rows: 16, or 8 (store and add epilogues, M <= 16): a block takes 8 rows of W, and ssq_out has a
// row per 8 columns, [ceil(N/8)][64].
// next_weight, xg (may be null; with ssq_out): the weight [N] (float) of the norm that follows, and
// where bfloat16(weight * x) of the completed rows goes, [M][ldxg].
// bias (may be null): N floats (gated: 2N), added to the sums; act: the gated epilogue's activation.
// w_tiled (may be null; N % 16 == 0): the same W as [strip of 16 rows][k-step of 32][lane][8 elements], k
// padded with zeros to whole steps (gated: the strips of the gate rows, then those of the up rows): the
// kernels that keep their rows of A in registers read W there.
// w_tiled8 (may be null; N % 8 == 0): W as [strip of 8 rows][step of 64 k][lane][8 elements], lane (r, q)
// holding row r % 8 at k = 32 (r / 8) + 8 q: the order of the packed tiles of strips of 8 rows (M <= 8).
// a_packed (strip_rows 8, M <= 8): A is not [M][lda] but the step's rows in that same order, [ceil(K / 64)][64][8],
// as a product with `pack_out` leaves them.
extern "C" int gl3_gemm_skinny(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, long lda,
                               long ldw, long ldc, int epilogue, int waves, float* ssq_out, int strip_rows,
                               const float* next_weight, void* xg, long ldxg, const float* bias, int act,
                               const void* w_tiled, const void* w_tiled8, int a_packed, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (check_common("gl3_gemm_skinny", A, W, C, M, N, K, lda, ldw, waves)) return -1;
  GL3_REQUIRE(ldc >= N, "gl3_gemm_skinny: ldc too small");
  GL3_REQUIRE(epilogue >= 0 && epilogue <= 2, "gl3_gemm_skinny: unknown epilogue %d", epilogue);
  GL3_REQUIRE(epilogue != SK_ADD || c_dtype == GL3_F32, "gl3_gemm_skinny: the add epilogue needs a float output");
  GL3_REQUIRE(!ssq_out || (epilogue == SK_ADD && N % 16 == 0),
              "gl3_gemm_skinny: sums of squares come with the add epilogue and N a multiple of 16");
  GL3_REQUIRE(strip_rows == 16 || (strip_rows == 8 && M <= 16 && epilogue != SK_GATED),
              "gl3_gemm_skinny: strips of %d rows (M=%d, epilogue %d)", strip_rows, M, epilogue);
  GL3_REQUIRE((next_weight == nullptr) == (xg == nullptr) && (!xg || (ssq_out && ldxg >= N)),
              "gl3_gemm_skinny: the next norm's weight and its rows come together, with the sums of squares");
  SkCall a = {A, W, C, M, N, K, lda, ldw, ldc, SkNorm{}, ssq_out, SkRope{}, stream, waves == 0, strip_rows};
  GL3_REQUIRE(act == GL3_ACT_SILU || act == GL3_ACT_GELU_TANH, "gl3_gemm_skinny: unknown activation %d", act);
  a.nx = SkNext{next_weight, (bf16_t*)xg, ldxg, bias, act, 0};
  GL3_REQUIRE(!w_tiled || (N % 16 == 0 && (uintptr_t)w_tiled % 16 == 0), "gl3_gemm_skinny: a copy of W in the operands' order needs N %% 16 == 0");
  a.Wt = w_tiled;
  GL3_REQUIRE(!w_tiled8 || (N % 8 == 0 && (uintptr_t)w_tiled8 % 16 == 0), "gl3_gemm_skinny: a copy of W in the packed tiles' order needs N %% 8 == 0");
  a.Wt8 = w_tiled8;
  GL3_REQUIRE(!a_packed || (strip_rows == 8 && M <= 8 && waves == 0 && epilogue != SK_GATED),
              "gl3_gemm_skinny: rows in the packed tiles' order are read by the strips of 8 rows with at most 8 rows of A");
  a.a_packed = a_packed;
  const int nw = pick_waves(waves, N, K);
  if (c_dtype == GL3_F32) {
    if (epilogue == SK_STORE) return pick_mt<SK_STORE, float, false, false>(nw, a);
    if (epilogue == SK_ADD) return ssq_out ? pick_mt<SK_ADD, float, false, true>(nw, a)
                                           : pick_mt<SK_ADD, float, false, false>(nw, a);
    return pick_mt<SK_GATED, float, false, false>(nw, a);
  } else if (c_dtype == GL3_BF16) {
    if (epilogue == SK_STORE) return pick_mt<SK_STORE, bf16_t, false, false>(nw, a);
    return pick_mt<SK_GATED, bf16_t, false, false>(nw, a);
  }
  GL3_REQUIRE(false, "gl3_gemm_skinny: unknown output dtype %d", c_dtype);
  return 0;
}

// The wide kernel addresses its operands with 32-bit byte offsets whose top bit means "nowhere".
static bool wide_addressable(long M, long w_rows, long K, long lda, long ldw) {
  return ((M - 1) * lda + K) * 2 < (1L << 31) && ((w_rows - 1) * ldw + K) * 2 < (1L << 31);
}

template <int MT, int NS, int EPI, typename TC, bool XNORM = false>
static int launch_wide(const SkCall& a, int slices, long slice_stride) {
  constexpr int NW = 8;
  const int n_strips = (a.N + 15) / 16;
  const int pairs = (a.K + 63) / 64;   // pairs of k-steps
  const int per_slice = (pairs + slices - 1) / slices;
  gemm_skinny_wide_kernel<MT, NS, NW, EPI, TC, XNORM>
      <<<dim3((n_strips + NS - 1) / NS, slices), dim3(NW * 64), 0, a.stream>>>(
          (const bf16_t*)a.A, (const bf16_t*)a.W, (TC*)a.C, a.M, a.N, a.K, a.lda, a.ldw, a.ldc, slice_stride, per_slice,
          a.rp, a.nx, a.nrm);
  GL3_LAUNCH_CHECK();
  return 0;
}

template <int EPI, typename TC>
static int pick_wide(const SkCall& a, int strips_per_block, int slices, long slice_stride) {
  constexpr int BIG = (EPI == SK_GATED) ? 2 : 4;   // a gated strip is a pair of strips
  const bool big = strips_per_block == BIG;
  if constexpr (EPI == SK_STORE && std::is_same<TC, float>::value) {   // (9 to 16 rows: slices of a long K only)
    if (a.M <= 16)
      return big ? launch_wide<1, BIG, EPI, TC>(a, slices, slice_stride)
                 : launch_wide<1, BIG / 2, EPI, TC>(a, slices, slice_stride);
  }
  if ((a.M + 15) / 16 <= 2)
    return big ? launch_wide<2, BIG, EPI, TC>(a, slices, slice_stride)
               : launch_wide<2, BIG / 2, EPI, TC>(a, slices, slice_stride);
  if ((a.M + 15) / 16 <= 3)
    return big ? launch_wide<3, BIG, EPI, TC>(a, slices, slice_stride)
               : launch_wide<3, BIG / 2, EPI, TC>(a, slices, slice_stride);
  return big ? launch_wide<4, BIG, EPI, TC>(a, slices, slice_stride)
             : launch_wide<4, BIG / 2, EPI, TC>(a, slices, slice_stride);
}

// How many strips a block of the wide kernel takes: as many as leave the chip enough blocks.
static int wide_strips(int N, int slices, int epilogue) {
  const int big = epilogue == SK_GATED ? 2 : 4;
  const long n_strips = (N + 15) / 16;
  return (n_strips / big) * slices >= 192 ? big : big / 2;
}

// The product for 17 to 64 rows of A (bfloat16), and for 9 to 16 with the store epilogue and a float
// output. `slices` > 1 (store epilogue, float output only):
// K is cut into that many slices and C is [slices][M][ldc] with `slice_stride` elements between
// slices; the caller adds them up. `strips_per_block`: 0 lets the library choose.
// bias (may be null; one slice only): N floats (gated: 2N); act: the gated epilogue's activation.
// ssq (may be null; gated epilogue, at most 16 rows, one slice): the product is that of RMSNorm(x), with A =
// bfloat16(norm weight * x) and the rows' sums of squares in `ssq` [n_partials][64], as gl3_gemm_skinny_norm takes
// them; pack_out (with ssq, at most 8 rows): C receives the rows in the packed tiles' order, as there.
extern "C" int gl3_gemm_skinny_wide(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, long lda,
                                    long ldw, long ldc, int epilogue, int slices, long slice_stride,
                                    int strips_per_block, const float* bias, int act, const float* ssq, int n_partials,
                                    float eps, int pack_out, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (check_common("gl3_gemm_skinny_wide", A, W, C, M, N, K, lda, ldw, 0)) return -1;
  GL3_REQUIRE(ssq || M > 16 || (M > 8 && epilogue == SK_STORE && c_dtype == GL3_F32),
              "gl3_gemm_skinny_wide: M=%d; up to 16 rows are gl3_gemm_skinny's (but 9 to 16 with a float output stored)", M);
  GL3_REQUIRE(!ssq || (M <= 16 && epilogue == SK_GATED && c_dtype == GL3_BF16 && slices == 1 && n_partials > 0),
              "gl3_gemm_skinny_wide: a folded norm goes with the gated epilogue, at most 16 rows and one slice");
  GL3_REQUIRE(!pack_out || (ssq && M <= 8), "gl3_gemm_skinny_wide: the packed tiles' order holds at most 8 rows of a folded norm's product");
  GL3_REQUIRE(wide_addressable(M, epilogue == SK_GATED ? 2L * N : N, K, lda, ldw),
              "gl3_gemm_skinny_wide: an operand of 2 GiB or more");
  GL3_REQUIRE(ldc >= N, "gl3_gemm_skinny_wide: ldc too small");
  GL3_REQUIRE(epilogue >= 0 && epilogue <= 2, "gl3_gemm_skinny_wide: unknown epilogue %d", epilogue);
  GL3_REQUIRE(slices >= 1 && slices <= (K + 63) / 64, "gl3_gemm_skinny_wide: %d slices of K=%d", slices, K);
  GL3_REQUIRE(slices == 1 || (epilogue == SK_STORE && c_dtype == GL3_F32 && slice_stride >= (long)(M - 1) * ldc + N),
              "gl3_gemm_skinny_wide: slices need the store epilogue, a float output and room for M rows a slice");
  GL3_REQUIRE(epilogue != SK_ADD || c_dtype == GL3_F32, "gl3_gemm_skinny_wide: the add epilogue needs a float output");
  const int big = epilogue == SK_GATED ? 2 : 4;
  if (strips_per_block == 0) {
    strips_per_block = wide_strips(N, slices, epilogue);
    // (a folded norm's product, one token tile: a block of two strip pairs stages 80 KB, so a CU holds one; more
    // than 256 of them would take a second round, where three blocks of one pair each fit a CU together.
    // N = 14,336, K = 4,096: 59 -> 49 us)
    if (ssq && ((N + 15) / 16 + 1) / 2 > 256) strips_per_block = 1;
  }
  GL3_REQUIRE(strips_per_block == big || strips_per_block == big / 2, "gl3_gemm_skinny_wide: %d strips per block",
              strips_per_block);
  GL3_REQUIRE(!bias || slices == 1, "gl3_gemm_skinny_wide: a bias goes with one slice of K");
  GL3_REQUIRE(act == GL3_ACT_SILU || act == GL3_ACT_GELU_TANH, "gl3_gemm_skinny_wide: unknown activation %d", act);
  SkCall a = {A, W, C, M, N, K, lda, ldw, ldc, SkNorm{ssq, n_partials, eps, nullptr}, nullptr, SkRope{}, stream, false};
  a.nx = SkNext{nullptr, nullptr, 0, bias, act, pack_out};
  if (ssq)
    return strips_per_block == big ? launch_wide<1, 2, SK_GATED, bf16_t, true>(a, 1, 0)
                                   : launch_wide<1, 1, SK_GATED, bf16_t, true>(a, 1, 0);
  if (c_dtype == GL3_F32) {
    if (epilogue == SK_STORE) return pick_wide<SK_STORE, float>(a, strips_per_block, slices, slice_stride);
    if (epilogue == SK_ADD) return pick_wide<SK_ADD, float>(a, strips_per_block, slices, slice_stride);
  } else if (c_dtype == GL3_BF16) {
    if (epilogue == SK_STORE) return pick_wide<SK_STORE, bf16_t>(a, strips_per_block, slices, slice_stride);
    if (epilogue == SK_GATED) return pick_wide<SK_GATED, bf16_t>(a, strips_per_block, slices, slice_stride);
  }
  GL3_REQUIRE(false, "gl3_gemm_skinny_wide: output dtype %d with epilogue %d is not built", c_dtype, epilogue);
  return 0;
}

// The product of RMSNorm(x) with W. xg: bfloat16(norm weight * x), [rows of x, K] (lda); ssq:
// [n_partials][64] partial sums of squares of the rows of x (indexed by the row of x, so x has at
// most 64 rows); `rows` (may be null) picks the rows of x that the product's rows read.
// Epilogues: store (float or bfloat16) and gated (bfloat16).
// bias (may be null): N floats (gated: 2N), added after the 1/rms; act: the gated epilogue's activation.
// pack_out (M <= 8, bfloat16): C is not [M][ldc] but the rows in the packed tiles' order (sk_packed_offset),
// [ceil(N / 64)][64][8], for a product of strips of 8 rows to read with `a_packed`.
extern "C" int gl3_gemm_skinny_norm(const void* xg, const int* rows, const float* ssq, int n_partials, float eps,
                                    const void* W, void* C, int c_dtype, int M, int N, int K, long lda, long ldw,
                                    long ldc, int epilogue, int waves, const float* bias, int act, const void* w_tiled,
                                    int pack_out, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (check_common("gl3_gemm_skinny_norm", xg, W, C, M, N, K, lda, ldw, waves)) return -1;
  GL3_REQUIRE(ssq && n_partials > 0, "gl3_gemm_skinny_norm: norm arguments missing");
  GL3_REQUIRE(ldc >= N, "gl3_gemm_skinny_norm: ldc too small");
  GL3_REQUIRE(epilogue == SK_STORE || epilogue == SK_GATED, "gl3_gemm_skinny_norm: epilogue %d", epilogue);
  GL3_REQUIRE(act == GL3_ACT_SILU || act == GL3_ACT_GELU_TANH, "gl3_gemm_skinny_norm: unknown activation %d", act);
  GL3_REQUIRE(!pack_out || (M <= 8 && c_dtype == GL3_BF16),
              "gl3_gemm_skinny_norm: the packed tiles' order holds at most 8 rows of bfloat16 (C then has 8 * 64 * ceil(N / 64) elements)");
  const SkNorm nrm = {ssq, n_partials, eps, rows};
  SkCall a = {xg, W, C, M, N, K, lda, ldw, ldc, nrm, nullptr, SkRope{}, stream, waves == 0};
  a.nx = SkNext{nullptr, nullptr, 0, bias, act, pack_out};
  GL3_REQUIRE(!w_tiled || (N % 16 == 0 && (uintptr_t)w_tiled % 16 == 0), "gl3_gemm_skinny_norm: a copy of W in the operands' order needs N %% 16 == 0");
  a.Wt = w_tiled;
  const int nw = pick_waves(waves, N, K);
  if (c_dtype == GL3_F32 && epilogue == SK_STORE) return pick_mt<SK_STORE, float, true, false>(nw, a);
  if (c_dtype == GL3_BF16 && epilogue == SK_STORE) return pick_mt<SK_STORE, bf16_t, true, false>(nw, a);
  if (c_dtype == GL3_BF16 && epilogue == SK_GATED) return pick_mt<SK_GATED, bf16_t, true, false>(nw, a);
  GL3_REQUIRE(false, "gl3_gemm_skinny_norm: output dtype %d with epilogue %d is not built", c_dtype, epilogue);
  return 0;
}

// a . Wqkv^T, rotation of q and k, q to `q_out` [M, n_heads*head_dim] (ldq), k and v into the paged
// cache (keys [page][kv head][position][head_dim], values transposed, in the tiles of gl3_k_offset
// and gl3_v_offset inside a page). One token per row; cos/sin
// null: no rotation. head_dim a multiple of 16; the rotation covers the whole head.
// ssq null: `a` holds the rows as they are. Else `a` is bfloat16(norm weight * x) and the product
// is that of RMSNorm(x), with the rows' sums of squares in `ssq` [n_partials][64].
extern "C" int gl3_qkv_rope_cache(const void* a_rows, const float* ssq, int n_partials, float eps, const void* Wqkv,
                                  void* q_out, long ldq, int M, int K, long lda, long ldw, const int* positions,
                                  const int* seq_of_token, const int* block_table, int table_stride,
                                  const float* cos_tab, const float* sin_tab, void* k_cache, void* v_cache,
                                  int n_heads, int n_kv, int head_dim, int adjacent, int page_size, int waves,
                                  const void* w_tiled, hipStream_t stream) {
  if (M == 0) return 0;
  const int N = (n_heads + 2 * n_kv) * head_dim;
  if (check_common("gl3_qkv_rope_cache", a_rows, Wqkv, q_out, M, N, K, lda, ldw, waves)) return -1;
  GL3_REQUIRE(!ssq || n_partials > 0, "gl3_qkv_rope_cache: sums of squares without their count");
  GL3_REQUIRE(head_dim % 16 == 0 && n_heads > 0 && n_kv > 0, "gl3_qkv_rope_cache: head_dim %d must be a multiple of 16",
              head_dim);
  GL3_REQUIRE(positions && seq_of_token && block_table && k_cache && v_cache && page_size > 0 && table_stride > 0,
              "gl3_qkv_rope_cache: cache arguments missing");
  GL3_REQUIRE(page_size % 32 == 0, "gl3_qkv_rope_cache: the cache lies in tiles: page_size %d must be a multiple of 32", page_size);
  GL3_REQUIRE((cos_tab == nullptr) == (sin_tab == nullptr), "gl3_qkv_rope_cache: one table without the other");
  GL3_REQUIRE(ldq >= (long)n_heads * head_dim && ldq % 4 == 0 && (uintptr_t)q_out % 8 == 0,
              "gl3_qkv_rope_cache: q_out stride/alignment");
  const SkNorm nrm = {ssq, n_partials, eps, nullptr};
  const SkRope rp = {positions, seq_of_token, block_table, table_stride, cos_tab, sin_tab, (bf16_t*)k_cache,
                     (bf16_t*)v_cache, n_heads, n_kv, head_dim, adjacent, page_size};
  SkCall a = {a_rows, Wqkv, q_out, M, N, K, lda, ldw, ldq, nrm, nullptr, rp, stream, waves == 0};
  GL3_REQUIRE(!w_tiled || (uintptr_t)w_tiled % 16 == 0, "gl3_qkv_rope_cache: the copy of W must be 16-byte aligned");
  a.Wt = w_tiled;   // (its strips hold the rows that sk_strip_row names: for half-split pairing 8 rows and the 8 half a head further)
  if (!ssq && waves == 0 && M > 16 && wide_addressable(M, N, K, lda, ldw)) {
    // many rows, read in whole lines: two strips a block, so that the rows are read half as often, where one
    // strip a block would be more blocks than CUs (N = 3,072, K = 2,048, 64 rows: 10.0 us with two, 8.9 us with
    // one; N = 5,120, K = 3,072: 16.3 against 20.7 us)
    const int tiles = (M + 15) / 16;
    if ((N + 15) / 16 <= 256)
      return tiles <= 2   ? launch_wide<2, 1, SK_QKV, bf16_t>(a, 1, 0)
             : tiles == 3 ? launch_wide<3, 1, SK_QKV, bf16_t>(a, 1, 0)
                          : launch_wide<4, 1, SK_QKV, bf16_t>(a, 1, 0);
    return tiles <= 2   ? launch_wide<2, 2, SK_QKV, bf16_t>(a, 1, 0)
           : tiles == 3 ? launch_wide<3, 2, SK_QKV, bf16_t>(a, 1, 0)
                        : launch_wide<4, 2, SK_QKV, bf16_t>(a, 1, 0);
  }
  if (!ssq) return pick_mt<SK_QKV, bf16_t, false, false>(pick_waves(waves, N, K), a);
  return pick_mt<SK_QKV, bf16_t, true, false>(pick_waves(waves, N, K), a);
}

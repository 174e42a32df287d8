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

// Time stamps inside a kernel, for measurements (compiled in with -DSK_STAMPS only, never in the library's own
// build): stage i of wave w (0 or the last) of block b (0 or the middle one) goes to sk_stamps[b][w][i].
#ifdef SK_STAMPS
__device__ long long sk_stamps[2][2][16];
extern "C" int gl3_sk_stamps(long long* out) {
  return hipMemcpyFromSymbol(out, HIP_SYMBOL(sk_stamps), sizeof(sk_stamps)) == hipSuccess ? 0 : -1;
}
#define SK_STAMP(i)                                                                                              \
  do {                                                                                                           \
    const int w_ = threadIdx.x >> 6, nw_ = blockDim.x >> 6;                                                      \
    if ((blockIdx.x == 0 || blockIdx.x == gridDim.x / 2) && (threadIdx.x & 63) == 0 && (w_ == 0 || w_ == nw_ - 1)) \
      sk_stamps[blockIdx.x == 0 ? 0 : 1][w_ == 0 ? 0 : 1][i] = (i) == 0 || (i) == 15 ? wall_clock64() : clock64(); \
  } while (0)
#else
#define SK_STAMP(i) do {} while (0)
#endif

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
  // what hangs on a token's position, looked up once per step for all layers (gl3_token_facts; may be null):
  // the page its keys and values go to, and its row of cos and sin, [tokens][head_dim]: cos, then sin
  const int* token_pages;
  const float* token_rot;
};

// Which row of W is row r of a strip's tile, and for SK_QKV which head the strip belongs to.
// A strip is ROWS rows of W: 16, or 8 (then rows 8..15 of the tile repeat rows 0..7 and are not
// written: half a tile is wasted for twice as many blocks where 16-row strips leave CUs idle).
// sk_strip_head is what costs (a division), once per strip; sk_strip_row_of is the row of one lane.
template <int EPI>
__device__ __forceinline__ void sk_strip_head(int strip, const SkRope& rp, int& hd, int& sub, bool& rotated) {
  hd = 0; sub = 0; rotated = false;
  if (EPI == SK_QKV) {
    const int per_head = rp.head_dim / 16;
    hd = strip / per_head;
    sub = strip - hd * per_head;
    rotated = rp.cos_tab != nullptr && hd < rp.n_heads + rp.n_kv;
  }
}
template <int EPI, int ROWS = 16>
__device__ __forceinline__ int sk_strip_row_of(int strip, int r, int N, const SkRope& rp, int hd, int sub, bool rotated) {
  if (EPI == SK_QKV && rotated && !rp.adjacent) return hd * rp.head_dim + 8 * sub + (r < 8 ? r : rp.head_dim / 2 + r - 8);
  return min(strip * ROWS + (r % ROWS), N - 1);
}
template <int EPI, int ROWS = 16>
__device__ __forceinline__ int sk_strip_row(int strip, int r, int N, const SkRope& rp, int& hd, int& sub, bool& rotated) {
  sk_strip_head<EPI>(strip, rp, hd, sub, rotated);
  return sk_strip_row_of<EPI, ROWS>(strip, r, N, rp, hd, sub, rotated);
}

// ---- loads without branches. Everything a block reads before its first product is asked for in one go, so
// that it arrives in one trip to memory. A branch around a load defeats that: at the point where the
// branches meet again the compiler waits for all loads on their way, and a prologue of conditional loads
// becomes a chain of trips (nine of them before the first matrix instruction of the QKV product, as
// compiled). So every load here goes through a buffer descriptor and is always issued: a lane that has
// nothing to read gives an offset beyond the buffer (SK_NOWHERE always is), gets zeros and touches no
// memory, and a null pointer makes an empty buffer.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr unsigned SK_NOWHERE = 0x80000000u;   // beyond any buffer: descriptors span less than 2 GiB

__device__ __forceinline__ __amdgpu_buffer_rsrc_t sk_rsrc(const void* p, long bytes) {
  const long n = p ? (bytes < 0x7fffffffL ? bytes : 0x7fffffffL) : 0;
  return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, (int)n, 0x00020000);
}
__device__ __forceinline__ bf16x8 sk_ld_b128(__amdgpu_buffer_rsrc_t buf, unsigned byte_offset) {
  return __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(buf, byte_offset, 0, 0));
}
__device__ __forceinline__ f32x4 sk_ld_f32x4(__amdgpu_buffer_rsrc_t buf, unsigned byte_offset) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(buf, byte_offset, 0, 0));
}
__device__ __forceinline__ float sk_ld_f32(__amdgpu_buffer_rsrc_t buf, unsigned byte_offset) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(buf, byte_offset, 0, 0));
}
__device__ __forceinline__ int sk_ld_i32(__amdgpu_buffer_rsrc_t buf, unsigned byte_offset) {
  return (int)__builtin_amdgcn_raw_buffer_load_b32(buf, byte_offset, 0, 0);
}
// 4 floats at element `first` of a float array of `count` elements; elements from `count` on read as zero.
// (Single loads: the array may start anywhere.)
__device__ __forceinline__ f32x4 sk_ld_4f(__amdgpu_buffer_rsrc_t buf, bool wanted, int first, int count) {
  f32x4 v;
#pragma unroll
  for (int c = 0; c < 4; ++c) v[c] = sk_ld_f32(buf, (wanted && first + c < count) ? (unsigned)(first + c) * 4u : SK_NOWHERE);
  return v;
}

// The row of A that row m of the product reads (XNORM with `rows`: the product is one of chosen rows). Called
// before anything else is on its way: the value is used at once, and the wait for it waits for nothing else.
template <bool XNORM>
__device__ __forceinline__ int sk_a_row(int m, int M, const SkNorm& nrm) {
  int row = min(m, M - 1);
  if (XNORM && nrm.rows) {   // (the same for the whole grid)
    row = nrm.rows[row];
    asm volatile("" : "+v"(row));
  }
  return row;
}

// Rows of A as [rows][lda] bfloat16 behind a descriptor; a row's offset is SK_NOWHERE when the row does not
// exist, so that its lanes ask for nothing: a CU draws a bounded number of bytes a second through its
// first-level cache, whatever they are.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t sk_a_rsrc(const void* Av, int M, int K, long lda, const SkNorm* nrm) {
  const long rows = (nrm && nrm->rows) ? 64 : M;   // (chosen rows: A has at most 64; offsets of rows that exist are all that is asked for)
  return sk_rsrc(Av, ((rows - 1) * lda + K) * 2);
}
__device__ __forceinline__ unsigned sk_x_off(int row, bool exists, long lda) {
  return exists ? (unsigned)((long)row * lda * 2) : SK_NOWHERE;
}
// A operands of one k-step for MT token tiles: elements k .. k+7 of each tile's row (`kb`: 2 k, or SK_NOWHERE).
template <int MT>
__device__ __forceinline__ void sk_load_x(bf16x8 (&xf)[MT], __amdgpu_buffer_rsrc_t a_buf, const unsigned (&xo)[MT], unsigned kb) {
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xf[mt] = sk_ld_b128(a_buf, ((xo[mt] | kb) & SK_NOWHERE) ? SK_NOWHERE : xo[mt] + kb);
}

// Partial sums of squares of the rows, added up in a fixed order: sm_ssq[w][row] receives wave w's share, the
// strip's end adds the waves' shares. `sq_row`: the lane's row's row of A (the partial sums are stored by it).
// One token tile (at most 16 rows, every decode step that folds a norm): the lanes are 4 groups of 16 rows, group j
// of wave w takes the partials w + NW (4 i + j), and the first four of each lane (64 NW partials in all) are
// asked for with the block's first loads (sk_ssq_ask); sk_ssq_sum, at the first strip's end, adds them, fetches
// any further ones, and adds the groups. More token tiles: lane = row, sixteen partials at a time, all in sk_ssq_sum.
// (SK_SQN: how many a lane asks for at the start: 512 partial sums a block, what strips of 8 columns of rows of 4,096 leave)
#define SK_SQN(NW) (128 / (NW))
template <int NW, int MT>
__device__ __forceinline__ void sk_ssq_ask(float (&sq)[SK_SQN(NW)], int M, const SkNorm& nrm, int sq_row) {
  if (MT != 1) return;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const __amdgpu_buffer_rsrc_t buf = sk_rsrc(nrm.ssq, (long)nrm.n_partials * 256);
#pragma unroll
  for (int i = 0; i < SK_SQN(NW); ++i) {
    const int p = wave + NW * (4 * i + (lane >> 4));
    sq[i] = sk_ld_f32(buf, ((lane & 15) < M && p < nrm.n_partials) ? (unsigned)((p * 64 + sq_row) * 4) : SK_NOWHERE);
  }
}
// `after`: a result of the product's matrix instructions. The sums are wanted at the strip's end; tied to that
// value they cannot be added up, and waited for, at the point where they were asked for, in front of loads
// that should be on their way first.
template <int NW, int MT>
__device__ __forceinline__ void sk_ssq_sum(float (*sm_ssq)[64], float (&sq)[SK_SQN(NW)], int M, const SkNorm& nrm, int sq_row,
                                           float after) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const __amdgpu_buffer_rsrc_t buf = sk_rsrc(nrm.ssq, (long)nrm.n_partials * 256);
  float sp = 0.f;
  if (MT == 1) {
    asm volatile("" : "+v"(sq[0]) : "v"(after));
#pragma unroll
    for (int i = 0; i < SK_SQN(NW); ++i) sp += sq[i];
    for (int p0 = wave + NW * 4 * SK_SQN(NW); p0 < nrm.n_partials; p0 += NW * 16) {   // further partial sums, four a lane at a time
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int p = p0 + NW * (4 * i + (lane >> 4));
        v[i] = sk_ld_f32(buf, ((lane & 15) < M && p < nrm.n_partials) ? (unsigned)((p * 64 + sq_row) * 4) : SK_NOWHERE);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) sp += v[i];
    }
    sp += __shfl_xor(sp, 16, 64);
    sp += __shfl_xor(sp, 32, 64);
  } else {
    for (int p0 = wave; p0 < nrm.n_partials; p0 += NW * 16) {
      float v[16];   // sixteen loads in flight, then added in order
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int p = p0 + NW * i;
        v[i] = sk_ld_f32(buf, (lane < M && p < nrm.n_partials) ? (unsigned)((p * 64 + sq_row) * 4) : SK_NOWHERE);
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

// A block's prologue is what its time goes to before the loads are on their way: sixteen waves that each work
// through several hundred instructions, most of them scalar, share one scalar unit. So what only the END of a
// strip needs (sk_token, sk_preload) is computed by the waves that finish a token tile alone (wave < MT: the
// caller's branch, the same for a whole wave), and offsets are 32-bit (the entry points bound the sizes).
//
// A token's position and its row of the block table (SK_QKV), asked for before the product's own loads so
// that what hangs on them (page number, cos and sin) can be asked for while those are still on their way.
struct SkToken { int pos, row; };
__device__ __forceinline__ SkToken sk_token(int M, const SkRope& rp, int tile = -1) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), r = threadIdx.x & 15;
  const int m = (tile < 0 ? wave : tile) * 16 + r;
  const unsigned at = m < M ? (unsigned)m * 4u : SK_NOWHERE;
  SkToken t;
  t.pos = sk_ld_i32(sk_rsrc(rp.positions, (long)M * 4), at);
  t.row = sk_ld_i32(sk_rsrc(rp.seq_of_token, (long)M * 4), at);
  return t;
}

// For a wave that finishes token tile `wave` (the caller sees to wave < MT). SK_QKV: `tok` is what sk_token
// returned. No branch surrounds a load: see sk_rsrc.
template <int MT, int EPI, typename TC, int ROWS = 16>
__device__ __forceinline__ SkPre sk_preload(const TC* __restrict__ C, int M, int N, long ldc, int strip, int hd, int sub,
                                            bool rotated, const SkRope& rp, const SkNext& nx = SkNext{},
                                            SkToken tok = SkToken{0, 0}, int tile = -1) {
  SkPre p;
  p.prev = p.bias = p.bias_up = p.next_w = p.co = p.si = f32x4{0.f, 0.f, 0.f, 0.f};
  p.pos = 0; p.page = 0;
  // (What is computed here is for the calling waves alone. Much of it does not change from strip to strip, and
  // the compiler would move that in front of the caller's loop over the strips, where every wave pays for it:
  // the values it all hangs on pass through an empty volatile statement, which stays where it is.)
  asm volatile("" : "+v"(tok.pos), "+v"(tok.row), "+s"(strip));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int m = (tile < 0 ? wave : tile) * 16 + r;   // (`tile`: the token tile that the wave finishes, its own number unless said)
  const bool live = m < M && 4 * q < ROWS;
  const int n = strip * ROWS + 4 * q;
  if (EPI != SK_QKV && nx.bias) {   // (the same for the whole grid; nothing hangs on these loads before the strip's end)
    const __amdgpu_buffer_rsrc_t b_buf = sk_rsrc(nx.bias, (long)(EPI == SK_GATED ? 2 * N : N) * 4);
    p.bias = sk_ld_4f(b_buf, live, n, N);
    if (EPI == SK_GATED) {
#pragma unroll
      for (int c = 0; c < 4; ++c) p.bias_up[c] = sk_ld_f32(b_buf, (live && n + c < N) ? (unsigned)(N + n + c) * 4u : SK_NOWHERE);
    }
  }
  if (EPI == SK_ADD) {
    static_assert(EPI != SK_ADD || sizeof(TC) == 4, "the add epilogue adds into a float matrix");
    const __amdgpu_buffer_rsrc_t c_buf = sk_rsrc(C, ((long)(M - 1) * ldc + N) * 4);
    const unsigned at = ((unsigned)m * (unsigned)ldc + (unsigned)n) * 4u;
#pragma unroll
    for (int c = 0; c < 4; ++c) p.prev[c] = sk_ld_f32(c_buf, (live && n + c < N) ? at + 4u * c : SK_NOWHERE);
    p.next_w = sk_ld_4f(sk_rsrc(nx.weight, (long)N * 4), live, n, N);
  }
  if (EPI == SK_QKV) {
    p.pos = tok.pos;
    // (the tables' sizes are not known here: the descriptors span what a descriptor can, and only lanes of
    // tokens that exist, whose entries the caller vouches for, give an offset inside)
    const bool kv = live && hd >= rp.n_heads;
    const unsigned half = (unsigned)rp.head_dim / 2u;
    const bool turn = live && rotated;
    const int pairs = rp.adjacent ? 2 : 4;                                                    // (the same for the whole grid)
    const unsigned pair0 = rp.adjacent ? (16u * sub + 4u * q) / 2u : 8u * sub + 4u * (q & 1);
    if (rp.token_pages) {   // (the same for the whole grid) looked up once per step: nothing here waits for the position
      p.page = sk_ld_i32(sk_rsrc(rp.token_pages, (long)M * 4), kv ? (unsigned)m * 4u : SK_NOWHERE);
      const __amdgpu_buffer_rsrc_t rot_buf = sk_rsrc(rp.token_rot, (long)M * rp.head_dim * 4);
      const unsigned at = ((unsigned)m * (unsigned)rp.head_dim + pair0) * 4u;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        p.co[c] = sk_ld_f32(rot_buf, (turn && c < pairs) ? at + 4u * c : SK_NOWHERE);
        p.si[c] = sk_ld_f32(rot_buf, (turn && c < pairs) ? at + (half + c) * 4u : SK_NOWHERE);
      }
    } else {
      const unsigned page_at = (unsigned)tok.row * (unsigned)rp.table_stride + (unsigned)tok.pos / (unsigned)rp.page_size;
      p.page = sk_ld_i32(sk_rsrc(rp.block_table, 0x7fffffffL), kv ? page_at * 4u : SK_NOWHERE);
      const __amdgpu_buffer_rsrc_t co_buf = sk_rsrc(rp.cos_tab, 0x7fffffffL), si_buf = sk_rsrc(rp.sin_tab, 0x7fffffffL);
      const unsigned at = ((unsigned)tok.pos * half + pair0) * 4u;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        p.co[c] = sk_ld_f32(co_buf, (turn && c < pairs) ? at + 4u * c : SK_NOWHERE);
        p.si[c] = sk_ld_f32(si_buf, (turn && c < pairs) ? at + 4u * c : SK_NOWHERE);
      }
    }
  }
  return p;
}

// The end of one token tile of a strip, by one wave: `v` (gated: and `up`) are the strip's sums for token tile `mt`,
// a lane holding tile rows 4q .. 4q+3 (columns of C) of token mt*16 + r. `sub`, `hd`, `rotated` describe the strip
// for SK_QKV; `pre` is what sk_preload asked for.
template <int MT, int NW, int EPI, typename TC, bool XNORM, bool SSQ, int ROWS = 16>
__device__ __forceinline__ void sk_end_tile(f32x4 v, f32x4 up, int mt, float (*sm_ssq)[64], int strip, int hd, int sub,
                                            bool rotated, TC* __restrict__ C, int M, int N, int K, long ldc,
                                            const SkNorm& nrm, float* __restrict__ ssq_out, const SkRope& rp,
                                            const SkNext& nx, const SkPre& pre) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int n0 = strip * ROWS;
  const int m = mt * 16 + r;
  const bool m_ok = m < M;
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
    return;
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
  SK_STAMP(6);
  for (int t = wave; t < NG * MT; t += NW) {
    f32x4 v = red[0][t][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) v += red[w][t][lane];
    red[0][t][lane] = v;   // only this thread touches red[*][t][lane] before the barrier
  }
  __syncthreads();
  SK_STAMP(7);

  // epilogue: lane holds tile rows 4q .. 4q+3 (columns of C) of token mt*16 + r
  for (int mt = wave; mt < MT; mt += NW)
    sk_end_tile<MT, NW, EPI, TC, XNORM, SSQ, ROWS>(red[0][mt][lane], (EPI == SK_GATED) ? red[0][MT + mt][lane] : zero4, mt, sm_ssq,
                                                   strip, hd, sub, rotated, C, M, N, K, ldc, nrm, ssq_out, rp, nx, pre);
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
  SK_STAMP(0); SK_STAMP(1);
  const int strip = blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  // which rows of A the tiles' rows are (a look-up for chosen rows), before anything else is on its way
  unsigned xo[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {   // nowhere for rows that do not exist: their lanes ask for nothing
    const int m = PACK ? (r & 7) : mt * 16 + r;
    xo[mt] = sk_x_off(sk_a_row<XNORM>(m, M, nrm), m < M, lda);
  }
  const int sq_row = XNORM ? sk_a_row<XNORM>(MT == 1 ? (lane & 15) : lane, M, nrm) : 0;
  const bool ender = wave < MT;   // this wave finishes token tile `wave`
  SkToken tok = {0, 0};
  if (EPI == SK_QKV && ender) tok = sk_token(M, rp);
  int hd, sub;
  bool rotated;
  const int wr = sk_strip_row<EPI, ROWS>(strip, r, N, rp, hd, sub, rotated);
  const int w0 = sk_strip_row_of<EPI, ROWS>(strip, 0, N, rp, hd, sub, rotated);   // the strip's first row: the same for the block
  const int koff = PACK ? 32 * (r >> 3) + q * 8 : q * 8;   // the lane's place inside a k-step
  const int steps = (K + 31) / 32;   // k-steps of 32
  const int steps64 = (K + 63) / 64;
  // W behind descriptors that start at the strip: as it is stored (the lane's row, 16 bytes at its place in
  // a k-step), or the copy in the order of the operands (Wt8: strips of 16 rows [strip][k-step of 32][lane][8],
  // gated: the up strips follow the N / 16 gate strips; PACK: [strip of 8 rows][step of 64 k][lane][8]; k
  // padded with zeros to whole steps), where a load is 1 KB of consecutive memory.
  const bool tiled = Wt8 != nullptr && (PACK || ROWS == 16);
  const long tile_bytes = PACK ? (long)steps64 * 1024 : (long)steps * 1024;
  const __amdgpu_buffer_rsrc_t w_buf =
      tiled ? sk_rsrc(Wt8 + (long)strip * (tile_bytes / 2), tile_bytes)
            : sk_rsrc(W + (long)w0 * ldw, (((long)(EPI == SK_QKV ? N : min(N, (strip + 1) * ROWS)) - 1 - w0) * ldw + K) * 2);
  const __amdgpu_buffer_rsrc_t u_buf =   // up rows (gated only)
      tiled ? sk_rsrc(Wt8 + ((long)(N / 16) + strip) * (tile_bytes / 2), tile_bytes)
            : sk_rsrc(W + ((long)N + w0) * ldw, (((long)min(N, (strip + 1) * ROWS) - 1 - w0) * ldw + K) * 2);
  const unsigned w_lane = tiled ? (unsigned)lane * 16u : (unsigned)(((long)(wr - w0) * ldw + koff) * 2);
  const unsigned w_step = tiled ? 1024u : (PACK ? 128u : 64u);   // bytes from one step to the next
  const __amdgpu_buffer_rsrc_t a_buf = a_packed ? sk_rsrc(Av, (long)steps64 * 1024) : sk_a_rsrc(Av, M, K, lda, XNORM ? &nrm : nullptr);
  float sq[SK_SQN(NW)];
  if (XNORM) sk_ssq_ask<NW, MT>(sq, M, nrm, sq_row);
  SkPre pre;
  if (ender) pre = sk_preload<MT, EPI, TC, ROWS>(C, M, N, ldc, strip, hd, sub, rotated, rp, nx, tok);
  SK_STAMP(2);

  f32x4 acc[NG][MT];
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[g][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  if (PACK) {
    // a wave takes steps of 64 k: step wave, wave + NW, ...
    for (int p0 = wave; p0 * 64 < K; p0 += NW * UNROLL) {
      bf16x8 wf[UNROLL], xf[UNROLL][MT];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int p = p0 + NW * u, k = p * 64;
        const bool ok = k + koff < K;   // K is a multiple of 8: a lane's 8 elements are all in or all out
        wf[u] = sk_ld_b128(w_buf, (tiled ? p < steps64 : ok) ? w_lane + (unsigned)p * w_step : SK_NOWHERE);
        // (a_packed: the rows in the packed tiles' order, sk_packed_offset: this lane's 16 bytes of step p)
        const unsigned at = a_packed ? (unsigned)(p * 64 + lane) * 16u : xo[0] + (unsigned)(k + koff) * 2u;
        xf[u][0] = sk_ld_b128(a_buf, (ok && (r & 7) < M) ? at : SK_NOWHERE);
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
  for (int p0 = wave; 2 * p0 < steps; p0 += NW * (UNROLL / 2)) {
    bf16x8 wf[UNROLL], uf[UNROLL], xf[UNROLL][MT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int st = 2 * (p0 + NW * (u / 2)) + (u & 1), k = st * 32;
      const bool ok = k + q * 8 < K;   // K is a multiple of 8: a lane's 8 elements are all in or all out
      const bool w_ok = tiled ? st < steps : ok;
      wf[u] = sk_ld_b128(w_buf, (w_ok && r < ROWS) ? w_lane + (unsigned)st * w_step : SK_NOWHERE);   // rows of the tile beyond the strip stay zero
      if (EPI == SK_GATED) uf[u] = sk_ld_b128(u_buf, w_ok ? w_lane + (unsigned)st * w_step : SK_NOWHERE);
      sk_load_x<MT>(xf[u], a_buf, xo, ok ? (unsigned)(k + q * 8) * 2u : SK_NOWHERE);
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
#ifdef SK_STAMPS
  asm volatile("s_nop 0" :: "v"(acc[0][0][0]));
  SK_STAMP(4);
#endif
  if (XNORM) sk_ssq_sum<NW, MT>(sm_ssq, sq, M, nrm, sq_row, acc[0][0][0]);
  SK_STAMP(5);
  sk_finish<MT, NW, EPI, TC, XNORM, SSQ, ROWS>(red, sm_ssq, acc, strip, hd, sub, rotated, C, M, N, K, ldc, nrm, ssq_out, rp,
                                               nx, pre);
  SK_STAMP(9); SK_STAMP(15);
}

// The packed strips of 8 rows (PACK above) over the copy of W in their own order, with the prologue cut down to
// what the loads' addresses take (see gemm_skinny_decode_kernel): the output and down projections of a decode
// step of at most 8 rows. A: the step's rows as they are, [M][lda], or in the packed tiles' order (`a_packed`).
// No test whether a step of W or a row of A exists: the descriptors end where the data ends, so a load beyond it
// reads zeros; a step that does not exist for the whole wave is not asked for at all. Elements of A from K on are
// not read (what lies there need not be a number, and the zeros of W that it would meet do not make it one).
template <int NW, int EPI, typename TC, bool SSQ>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_pack_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ Wt8,
                                                                   TC* __restrict__ C, int M, int N, int K, int lda, long ldc,
                                                                   float* __restrict__ ssq_out, SkNext nx, int a_packed) {
  constexpr int UNROLL = 8, MT = 1;
  __shared__ f32x4 red[NW][1][64];
  __shared__ float sm_ssq[1][64];
  SK_STAMP(0); SK_STAMP(1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int strip = blockIdx.x;
  const int steps64 = (K + 63) >> 6;
  const unsigned tile_bytes = (unsigned)steps64 << 10;   // a strip of the copy: 1 KB a step of 64 k
  const __amdgpu_buffer_rsrc_t w_buf = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)Wt8 + (long)strip * tile_bytes), 0, (int)tile_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t a_buf = __builtin_amdgcn_make_buffer_rsrc(
      (void*)A, 0, a_packed ? (int)tile_bytes : (int)((((unsigned)M - 1u) * (unsigned)lda + (unsigned)K) * 2u), 0x00020000);
  const unsigned w_at = (unsigned)lane * 16u + (unsigned)wave * 1024u;
  // lane (r, q) holds row r % 8 at k = 64 p + 32 (r / 8) + 8 q; in the packed order that is the lane's own 16 bytes of step p
  const unsigned x_at = a_packed ? ((r & 7) < M ? w_at : SK_NOWHERE)
                                 : ((unsigned)(r & 7) * (unsigned)lda + 32u * (r >> 3) + 8u * q + (unsigned)wave * 64u) * 2u;
  const unsigned x_step = a_packed ? 1024u : 128u;
  const int k_lane = 32 * (r >> 3) + 8 * q;   // the lane's k inside a step (K is a multiple of 8: its 8 elements are all in or all out)
  SkPre pre;
  if (wave == 0) pre = sk_preload<MT, EPI, TC, 8>(C, M, N, ldc, strip, 0, 0, false, SkRope{}, nx);
  f32x4 acc[1][MT];
  acc[0][0] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // a wave takes steps of 64 k: step wave, wave + NW, ...
  for (int p0 = wave; p0 < steps64; p0 += NW * UNROLL) {
    bf16x8 wf[UNROLL], xf[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      wf[u] = zero; xf[u] = zero;
      if (p0 + NW * u < steps64) {   // (the same for the wave)
        const unsigned p = (unsigned)(p0 - wave + NW * u);
        wf[u] = sk_ld_b128(w_buf, w_at + p * 1024u);
        xf[u] = sk_ld_b128(a_buf, ((x_at & SK_NOWHERE) || 64 * (p0 + NW * u) + k_lane >= K) ? SK_NOWHERE : x_at + p * x_step);
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // all of the batch's loads are issued before the first is waited for
    SK_STAMP(2);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
      acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u], xf[u], acc[0][0], 0, 0, 0);
  }
  // lane (token column j, quarter q) holds tile rows 4q .. 4q+3: the sums over the first 32 k of every
  // step lie at j < 8, q < 2, those over the second at j >= 8, q >= 2: lane + 40
#pragma unroll
  for (int c = 0; c < 4; ++c) acc[0][0][c] += __shfl_xor(acc[0][0][c], 40, 64);
#ifdef SK_STAMPS
  asm volatile("s_nop 0" :: "v"(acc[0][0][0]));
  SK_STAMP(4); SK_STAMP(5);
#endif
  sk_finish<MT, NW, EPI, TC, false, SSQ, 8>(red, sm_ssq, acc, strip, 0, 0, false, C, M, N, K, ldc, SkNorm{}, ssq_out, SkRope{}, nx,
                                            pre);
  SK_STAMP(9); SK_STAMP(15);
}

// The resident kernel: K <= 32 * NW * KS. `n_strips` strips are shared out over the blocks.
template <int MT, int NW, int KS, int EPI, typename TC, bool XNORM, bool SSQ, int WO>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_resident_kernel(
    const void* __restrict__ Av, const bf16_t* __restrict__ W, TC* __restrict__ C, int M, int N, int K, long lda,
    long ldw, long ldc, SkNorm nrm, float* __restrict__ ssq_out, SkNext nx, SkRope rp, int n_strips,
    const bf16_t* __restrict__ Wt_) {
  // WO 1: W comes as the copy in the operands' order (Wt_); 0: as stored rows; 2: whichever Wt_ says, at run time.
  // (A template parameter: decided at run time, every load of every strip takes a branch, 250 to 400 of the kernel's
  // 800 to 1,070 instructions. Sixteen waves with eight k-steps each have no register to spare, and without those
  // branches the compiler asks for everything at once and spills: they keep the run-time form.)
  const bool WT = WO == 2 ? Wt_ != nullptr : WO == 1;
  const bf16_t* const Wt = WT ? Wt_ : nullptr;
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  __shared__ f32x4 red[NW][NG * MT][64];
  __shared__ float sm_ssq[XNORM ? NW : 1][64];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  SK_STAMP(0); SK_STAMP(1);
  const bool ender = wave < MT;   // this wave finishes token tile `wave` of every strip
  // The order below is the order of need: the token's position first (the longest chain hangs on it), then the
  // loads that every wave's matrix instructions wait for, with as few instructions in front of them as can be;
  // everything else (which head a strip belongs to, what the strip's end reads) while those are on their way.
  SkToken tok = {0, 0};
  if (EPI == SK_QKV && ender) tok = sk_token(M, rp);
  // which rows of A the tiles' rows are (a look-up for chosen rows)
  unsigned xo[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)   // nowhere for rows that do not exist: their lanes ask for nothing
    xo[mt] = sk_x_off(sk_a_row<XNORM>(mt * 16 + r, M, nrm), mt * 16 + r < M, lda);
  const int sq_row = XNORM ? sk_a_row<XNORM>(MT == 1 ? (lane & 15) : lane, M, nrm) : 0;
  // Where a strip's operands lie. In W itself a lane's 16 bytes of k-step s are in its row at 32 s
  // elements; every lane of a load is then on a line of its own. In the copy in the operands' own
  // order (Wt, may be null: [strip][k-step][lane][8], k padded with zeros to whole steps, the strips'
  // rows as sk_strip_row names them; gated: the up strips follow the N / 16 gate strips) a load is 1 KB of
  // consecutive memory, which the CU's first-level cache takes in less than half the time. Either way the
  // strip lies behind a descriptor that starts at its first row (see sk_rsrc).
  const int steps_all = (K + 31) / 32;
  const unsigned w_step = WT ? 1024u : 64u;                // bytes from one k-step to the next
  const long tile = (long)steps_all * 512;                 // elements of a strip of the copy
  struct Strip { __amdgpu_buffer_rsrc_t w, u; unsigned lane_at; };
  auto strip_at = [&](int strip_) {
    Strip t;
    if (WT) {
      t.w = sk_rsrc(Wt + strip_ * tile, tile * 2);
      t.u = sk_rsrc(Wt + ((long)(N / 16) + strip_) * tile, tile * 2);
      t.lane_at = (unsigned)lane * 16u;
    } else {
      int hd, sub;
      bool rotated;
      const int wr = sk_strip_row<EPI>(strip_, r, N, rp, hd, sub, rotated);
      const int w0 = sk_strip_row_of<EPI>(strip_, 0, N, rp, hd, sub, rotated);   // the strip's first row: the same for the block
      const long bytes = (((EPI == SK_QKV ? N : min(N, (strip_ + 1) * 16)) - w0 - 1) * ldw + K) * 2;
      t.w = sk_rsrc(W + (long)w0 * ldw, bytes);
      t.u = sk_rsrc(W + ((long)N + w0) * ldw, bytes);
      t.lane_at = ((unsigned)(wr - w0) * (unsigned)ldw + (unsigned)q * 8u) * 2u;
    }
    return t;
  };
  auto step_at = [&](const Strip& t, int st) {   // the offset of this lane's 16 bytes of k-step st
    return (WT ? st < steps_all : st * 32 + q * 8 < K) ? t.lane_at + (unsigned)st * w_step : SK_NOWHERE;
  };
  int strip = blockIdx.x;
  Strip cur = strip_at(strip);
  bf16x8 wf[KS], uf[KS];
#pragma unroll
  for (int i = 0; i < KS; ++i) {
    wf[i] = sk_ld_b128(cur.w, step_at(cur, wave + NW * i));
    if (EPI == SK_GATED) uf[i] = sk_ld_b128(cur.u, step_at(cur, wave + NW * i));
  }
  bf16x8 xf[KS][MT];
  {
    const __amdgpu_buffer_rsrc_t a_buf = sk_a_rsrc(Av, M, K, lda, XNORM ? &nrm : nullptr);
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const int k = (wave + NW * i) * 32 + q * 8;
      sk_load_x<MT>(xf[i], a_buf, xo, k < K ? (unsigned)k * 2u : SK_NOWHERE);
    }
  }
  float sq[SK_SQN(NW)];
  if (XNORM) sk_ssq_ask<NW, MT>(sq, M, nrm, sq_row);
  __builtin_amdgcn_sched_barrier(0);   // all of that is on its way before anything else is computed
  SK_STAMP(2);
  bool first_strip = true;
  while (strip < n_strips) {
    // what the strip's end reads, then the next strip's rows, both before this strip's rows are used: the
    // end then waits for its own loads only, and the next rows travel while this strip is finished
    int hd = 0, sub = 0;
    bool rotated = false;
    SkPre pre;
    if (ender) {
      sk_strip_head<EPI>(strip, rp, hd, sub, rotated);
      pre = sk_preload<MT, EPI, TC>(C, M, N, ldc, strip, hd, sub, rotated, rp, nx, tok);
    }
    const int next = strip + gridDim.x;
    Strip nxt = cur;
    bf16x8 wn[KS], un[KS];
    if (next < n_strips) {   // (the same for the block; what is loaded here is used after the strip's end)
      nxt = strip_at(next);
#pragma unroll
      for (int i = 0; i < KS; ++i) {
        wn[i] = sk_ld_b128(nxt.w, step_at(nxt, wave + NW * i));
        if (EPI == SK_GATED) un[i] = sk_ld_b128(nxt.u, step_at(nxt, wave + NW * i));
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // the next strip's loads are on their way before this strip's are used
    SK_STAMP(3);
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
#ifdef SK_STAMPS
    asm volatile("s_nop 0" :: "v"(acc[0][0][0]));
    SK_STAMP(4);
#endif
    if (XNORM && first_strip) {
      sk_ssq_sum<NW, MT>(sm_ssq, sq, M, nrm, sq_row, acc[0][0][0]);   // (read after the barrier before the first strip's end)
      first_strip = false;
    }
    SK_STAMP(5);
    sk_finish<MT, NW, EPI, TC, XNORM, SSQ>(red, sm_ssq, acc, strip, hd, sub, rotated, C, M, N, K, ldc, nrm, ssq_out, rp, nx,
                                           pre);
    SK_STAMP(9); SK_STAMP(15);
    if (next >= n_strips) break;
    __syncthreads();   // the partial tiles in shared memory are free again
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      wf[i] = wn[i];
      if (EPI == SK_GATED) uf[i] = un[i];
    }
    strip = next;
    cur = nxt;
  }
}

// The resident kernel for the products of a decode step proper: a folded norm in front (XNORM), at most 16 rows
// (one token tile), all of them in order, W as the copy in the operands' order. What it leaves out is the
// general kernel's choices at run time (which W, which rows), not work: a block's sixteen waves share the CU's
// one scalar unit, and before the loads are on their way every wave works through the same prologue; measured
// inside the QKV product of the 1B layers, the last of sixteen waves had its loads out 2.2 us after it started
// with the general prologue. Here the prologue is what the loads' addresses take and no more:
//  * no test whether a k-step or a partial sum exists. The descriptors end where the data ends (a strip of the
//    copy, the partial sums), so a load beyond it reads zeros: k-steps beyond K (the copy is padded with zeros to
//    whole steps; elements of A from K on are not read), partial sums from n_partials on;
//  * what only the end of a strip needs is computed by wave 0 alone, after the loads are out.
template <int NW, int KS, int EPI, typename TC>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_decode_kernel(
    const bf16_t* __restrict__ xg, const bf16_t* __restrict__ Wt, TC* __restrict__ C, int M, int N, int K, int lda,
    long ldc, SkNorm nrm, SkNext nx, SkRope rp, int n_strips) {
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  constexpr int MT = 1;
  __shared__ f32x4 red[NW][NG][64];
  __shared__ float sm_ssq[NW][64];
  SK_STAMP(0); SK_STAMP(1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const bool ender = wave == 0;
  SkToken tok = {0, 0};
  if (EPI == SK_QKV && ender) tok = sk_token(M, rp);
  // the row of A that the product's row r reads: r itself, or a chosen one (the head on the wanted rows)
  int a_row = r;
  if (nrm.rows) {   // (the same for the whole grid; nothing else is on its way yet)
    a_row = nrm.rows[min(r, M - 1)];
    asm volatile("" : "+v"(a_row));
  }
  const unsigned tile_bytes = (unsigned)((K + 31) >> 5) << 10;   // a strip of the copy: 1 KB a k-step
  const unsigned up_strips = (unsigned)N >> 4;                   // (gated) the up strips follow the gate strips
  int strip = blockIdx.x;
  const unsigned w_at = (unsigned)lane * 16u + (unsigned)wave * 1024u;
  bf16x8 wf[KS], uf[KS];
  {
    const __amdgpu_buffer_rsrc_t w_buf = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)Wt + (long)strip * tile_bytes), 0, (int)tile_bytes, 0x00020000);
#pragma unroll
    for (int i = 0; i < KS; ++i) wf[i] = sk_ld_b128(w_buf, w_at + (unsigned)i * (NW * 1024u));
    if (EPI == SK_GATED) {
      const __amdgpu_buffer_rsrc_t u_buf = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)Wt + (long)(up_strips + strip) * tile_bytes), 0, (int)tile_bytes, 0x00020000);
#pragma unroll
      for (int i = 0; i < KS; ++i) uf[i] = sk_ld_b128(u_buf, w_at + (unsigned)i * (NW * 1024u));
    }
  }
  bf16x8 xf[KS][MT];
  {
    // (A has at most 64 rows; only rows that exist give an offset)
    const __amdgpu_buffer_rsrc_t a_buf = __builtin_amdgcn_make_buffer_rsrc((void*)xg, 0, (int)((63u * (unsigned)lda + (unsigned)K) * 2u), 0x00020000);
    const unsigned k0 = (unsigned)wave * 32u + (unsigned)q * 8u;
    const unsigned x_at = r < M ? ((unsigned)a_row * (unsigned)lda + k0) * 2u : SK_NOWHERE;
#pragma unroll
    for (int i = 0; i < KS; ++i)
      xf[i][0] = sk_ld_b128(a_buf, (r < M && k0 + (unsigned)i * (NW * 32u) < (unsigned)K) ? x_at + (unsigned)i * (NW * 64u) : SK_NOWHERE);
  }
  float sq[SK_SQN(NW)];
  const __amdgpu_buffer_rsrc_t s_buf = __builtin_amdgcn_make_buffer_rsrc((void*)nrm.ssq, 0, nrm.n_partials * 256, 0x00020000);
  const unsigned s_at = ((unsigned)wave + (unsigned)q * NW) * 256u + (unsigned)a_row * 4u;   // partial wave + NW (4 i + q) of the row (they are stored by row of A)
#pragma unroll
  for (int i = 0; i < SK_SQN(NW); ++i) sq[i] = sk_ld_f32(s_buf, s_at + (unsigned)i * (NW * 1024u));
  __builtin_amdgcn_sched_barrier(0);   // all of that is on its way before anything else is computed
  SK_STAMP(2);
  bool first_strip = true;
  while (true) {
    int hd = 0, sub = 0;
    bool rotated = false;
    SkPre pre;
    if (ender) {
      sk_strip_head<EPI>(strip, rp, hd, sub, rotated);
      pre = sk_preload<MT, EPI, TC>(C, M, N, ldc, strip, hd, sub, rotated, rp, nx, tok);
    }
    const int next = strip + gridDim.x;
    bf16x8 wn[KS], un[KS];
    if (next < n_strips) {   // (the same for the block; what is loaded here is used after the strip's end)
      const __amdgpu_buffer_rsrc_t w_buf = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)Wt + (long)next * tile_bytes), 0, (int)tile_bytes, 0x00020000);
#pragma unroll
      for (int i = 0; i < KS; ++i) wn[i] = sk_ld_b128(w_buf, w_at + (unsigned)i * (NW * 1024u));
      if (EPI == SK_GATED) {
        const __amdgpu_buffer_rsrc_t u_buf = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)Wt + (long)(up_strips + next) * tile_bytes), 0, (int)tile_bytes, 0x00020000);
#pragma unroll
        for (int i = 0; i < KS; ++i) un[i] = sk_ld_b128(u_buf, w_at + (unsigned)i * (NW * 1024u));
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // the next strip's loads are on their way before this strip's are used
    SK_STAMP(3);
    f32x4 acc[NG][MT];
#pragma unroll
    for (int g = 0; g < NG; ++g) acc[g][0] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i], xf[i][0], acc[0][0], 0, 0, 0);
      if (EPI == SK_GATED) acc[1][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[i], xf[i][0], acc[1][0], 0, 0, 0);
    }
#ifdef SK_STAMPS
    asm volatile("s_nop 0" :: "v"(acc[0][0][0]));
    SK_STAMP(4);
#endif
    if (first_strip) {
      // the waves' shares of the rows' sums of squares (tied to a result of the matrix instructions: see sk_ssq_sum)
      // (the order of sk_ssq_sum, so that both kernels give the same sums)
      asm volatile("" : "+v"(sq[0]) : "v"(acc[0][0][0]));
      float sp = 0.f;
#pragma unroll
      for (int i = 0; i < SK_SQN(NW); ++i) sp += sq[i];
      for (int p0 = wave + NW * 4 * SK_SQN(NW); p0 < nrm.n_partials; p0 += NW * 16) {   // further partial sums, four a lane at a time
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = sk_ld_f32(s_buf, s_at + (unsigned)(p0 - wave) * 256u + (unsigned)i * (NW * 1024u));
#pragma unroll
        for (int i = 0; i < 4; ++i) sp += v[i];
      }
      sp += __shfl_xor(sp, 16, 64);
      sp += __shfl_xor(sp, 32, 64);
      sm_ssq[wave][lane] = sp;
      first_strip = false;
    }
    SK_STAMP(5);
    sk_finish<MT, NW, EPI, TC, true, false>(red, sm_ssq, acc, strip, hd, sub, rotated, C, M, N, K, ldc, nrm, nullptr, rp, nx, pre);
    SK_STAMP(9); SK_STAMP(15);
    if (next >= n_strips) break;
    __syncthreads();   // the partial tiles in shared memory are free again
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      wf[i] = wn[i];
      if (EPI == SK_GATED) uf[i] = un[i];
    }
    strip = next;
  }
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
template <int MT, int NS, int NW, int EPI, typename TC, bool XNORM, int WL>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_wide_kernel(const bf16_t* __restrict__ A,
                                                                   const bf16_t* __restrict__ W, TC* __restrict__ C,
                                                                   int M, int N, int K, long lda, long ldw, long ldc,
                                                                   long slice_stride, int pairs_per_slice, SkRope rp,
                                                                   SkNext nx, SkNorm nrm) {
  constexpr int wl = WL;   // (a template parameter: as a run-time value every tile of every pair took a branch and two copies)
  // wl: how W lies. 0: rows as they are stored. 1: the matrix operands' order alone, [strip of 16 rows][k-step of 32]
  // [lane][8] (lib.tile_weight; for the stacked q, k, v rows the strips hold the rows that sk_strip_row names).
  // 2: the packed strips of 8 rows, [strip of 8][step of 64 k][lane][8] (lib.tile_weight8). In both orders a lane can
  // load what it holds as the matrix instruction's operand straight from memory, in whole 128-byte lines (the
  // operands' order IS that layout; of the packed strips lane (r, q) takes row r % 8 of strip r / 8 at the k block q
  // of the k-step's half): the tiles of W then do not pass through shared memory at all, only the rows of A do.
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  constexpr int NWT = NS * NG;        // tiles of W a pair of k-steps
  constexpr int NT = NWT + MT;        // tiles a wave stages for a pair of k-steps: 16 rows x 128 bytes each
  SK_STAMP(0); SK_STAMP(1);
  constexpr int NTILES = NS * NG * MT;   // the partial tiles of a wave: all of the block's strips end together
  constexpr int STAGE = NW * NT * 2048, RED = NW * NTILES * 1024;
  __shared__ __attribute__((aligned(16))) char smem[STAGE > RED ? STAGE : RED];
  __shared__ float sm_ssq[XNORM ? NW : 1][64];
  f32x4 (*red)[NTILES][64] = (f32x4 (*)[NTILES][64])smem;   // the partial tiles, once the staging is over
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int l8 = lane >> 3, c8 = lane & 7;
  const int n_strips = (N + 15) / 16;
  const int strip0 = blockIdx.x * NS;
  SK_STAMP(10);
  char* stage = smem + wave * (NT * 2048);
  // where this lane's loads go inside a tile (rows l8 and 8 + l8) and where its operands lie (k-steps 0, 1)
  const int put0 = l8 * 128 + ((c8 ^ l8) * 16);
  const int put1 = (8 + ((l8 + 1) & 7)) * 128 + ((c8 ^ l8) * 16);
  const int line = r < 8 ? r : 8 + ((r + 1) & 7);
  const int get0 = line * 128 + ((q ^ (r & 7)) * 16);
  const int get1 = line * 128 + (((4 + q) ^ (r & 7)) * 16);
  // where the lane's two loads of a tile of W go: (row, 16-byte piece) is (l8, c8) and (8 + l8, c8) for stored rows,
  // (r, q) and (r, 4 + q) for a k-step of the operands' order each, (lane % 8 [+ 8], 4 * (lane / 8 % 2) + q) for the
  // packed strips of 8
  const int putw0 = put0, putw1 = put1;   // (stored rows: as the rows of A)

  // Both operands are read through buffer descriptors: a lane whose row or k does not exist gives
  // an offset beyond the buffer and gets zeros without a branch around the load, so every wave issues
  // the same loads in the same order and can wait for exactly the ones it needs.
  const unsigned strip_bytes = wl == 1 ? (unsigned)((K + 31) >> 5) << 10 : (unsigned)((K + 63) >> 6) << 10;   // (wl 1, 2)
  const long w_bytes = wl == 0 ? (((long)NG * N - 1) * ldw + K) * 2
                       : wl == 1 ? (long)NG * (N >> 4) * strip_bytes : (long)(N >> 3) * strip_bytes;
  const __amdgpu_buffer_rsrc_t w_buf = __builtin_amdgcn_make_buffer_rsrc((void*)W, 0, (int)w_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t a_buf =
      __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (int)((((long)M - 1) * lda + K) * 2), 0x00020000);
  constexpr unsigned NOWHERE = SK_NOWHERE;   // beyond any buffer the entry point lets in
  int hd[NS], sub[NS];
  bool rotated[NS];
  unsigned wo[NWT][2];   // byte offsets of this lane's lines at k = 0
#pragma unroll
  for (int g = 0; g < NS; ++g)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int strip_g = min(strip0 + g, n_strips - 1);
      const int wr = sk_strip_row<EPI>(strip_g, 8 * j + l8, N, rp, hd[g], sub[g], rotated[g]);
#pragma unroll
      for (int h = 0; h < NG; ++h)   // (32-bit: the entry point lets in operands below 2 GiB only)
        // (wl 1, 2: j is the k-step of the pair, and the lane's 16 bytes are its operand of that k-step)
        wo[g * NG + h][j] = wl == 0   ? ((unsigned)(wr + h * N) * (unsigned)ldw + (unsigned)c8 * 8u) * 2u
                            : wl == 1 ? (unsigned)(strip_g + h * (N >> 4)) * strip_bytes + (unsigned)j * 1024u + (unsigned)lane * 16u
                                      : (unsigned)(2 * strip_g + (r >> 3)) * strip_bytes + (unsigned)(2 * q + j) * 128u + (unsigned)(r & 7) * 16u;
    }
  unsigned xo[MT][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int m = mt * 16 + 8 * j + l8;
      xo[mt][j] = m < M ? ((unsigned)m * (unsigned)lda + (unsigned)c8 * 8u) * 2u : NOWHERE;
    }

  SK_STAMP(11);
  TC* out = C + (long)blockIdx.y * slice_stride;
  // The rotation's end needs the token's position, and through it a page number and cos and sin:
  // two trips to memory one after the other. The position is asked for before the first lines of the
  // product, what hangs on it right after them, so that both trips run beside the product's first.
  // wave w finishes the token tiles w, w + NW, ... of the block's NS * MT (tile i: token tile i % MT of strip i / MT)
  constexpr int ENDS = (NS * MT + NW - 1) / NW;
  const bool ender = wave < NS * MT;
  SkToken tok[ENDS];
#pragma unroll
  for (int e = 0; e < ENDS; ++e) {
    tok[e] = SkToken{0, 0};
    if (EPI == SK_QKV && wave + e * NW < NS * MT) tok[e] = sk_token(M, rp, (wave + e * NW) % MT);
  }
  const int sq_row = MT == 1 ? (lane & 15) : lane;   // (a folded norm's product of all rows, in order)
  float sq[SK_SQN(NW)];

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
  // chip asks for all parts of the rows of W and not for the same quarter of every row. Over the packed strips of
  // 8 (wl 2) a wave takes a run of neighbouring pairs instead: with pairs dealt out in turn a block's eight waves ask
  // for 8 KB in a row of each of its few strips at a time, with runs for 1 KB at eight places of each (the down
  // projection of the 1B layers at 16 rows: 11.2 -> 9.4 us, what the stored rows take). Stored rows and the
  // operands' order are the other way round: runs cost them 3%.
  const int n_it = (p_end - p_begin + NW - 1) / NW;
  // (any spread will do; a remainder by a number not known before costs some forty instructions in every wave)
  const int rot = (n_it & (n_it - 1)) == 0 ? (int)(blockIdx.x & (unsigned)(n_it - 1)) : (int)(((blockIdx.x & 255u) * (unsigned)n_it) >> 8);
  const bool blocked_pairs = wl == 2;
  auto pair_at = [&](int i) {   // (i >= n_it: past the end)
    const int j = i + rot;
    const int jj = j < n_it ? j : j - n_it;
    return i >= n_it ? p_end : blocked_pairs ? p_begin + wave * n_it + jj : p_begin + wave + NW * jj;
  };
  bf16x8 held[NT][2];
  const unsigned w_pair = wl == 0 ? 128u : wl == 1 ? 2048u : 1024u;   // bytes from one pair of k-steps to the next
  const int k_steps = (K + 31) >> 5;
  auto ask = [&](int p) {
    const unsigned k2 = (p < p_end && p * 64 + c8 * 8 < K) ? (unsigned)p * 128u : NOWHERE;   // (K is a multiple of 8)
    // (the copies are padded with zeros to whole steps; the operands' order may end after a pair's first k-step)
    const unsigned kw0 = wl == 0 ? k2 : p < p_end ? (unsigned)p * w_pair : NOWHERE;
    const unsigned kw1 = (wl == 1 && 2 * p + 1 >= k_steps) ? NOWHERE : kw0;
#pragma unroll
    for (int t = 0; t < NWT; ++t) {
      held[t][0] = sk_ld_b128(w_buf, wo[t][0] + kw0);   // (offsets are below 2^31: with NOWHERE added they are beyond any buffer)
      held[t][1] = sk_ld_b128(w_buf, wo[t][1] + kw1);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        held[NWT + mt][j] = sk_ld_b128(a_buf, ((xo[mt][j] | k2) & NOWHERE) ? NOWHERE : xo[mt][j] + k2);
  };
  SK_STAMP(12);
  ask(pair_at(0));
  SK_STAMP(2);
  SkPre pre[ENDS];
  int end_hd[ENDS], end_sub[ENDS];
  bool end_rot[ENDS];
#pragma unroll
  for (int e = 0; e < ENDS; ++e) {
    end_hd[e] = end_sub[e] = 0;
    end_rot[e] = false;
    if (wave + e * NW < NS * MT) {   // (the same for the wave)
      const int end_g = (wave + e * NW) / MT;
#pragma unroll
      for (int g = 0; g < NS; ++g)
        if (g == end_g) { end_hd[e] = hd[g]; end_sub[e] = sub[g]; end_rot[e] = rotated[g]; }
      pre[e] = sk_preload<MT, EPI, TC>(out, M, N, ldc, min(strip0 + end_g, n_strips - 1), end_hd[e], end_sub[e], end_rot[e], rp,
                                       nx, tok[e], (wave + e * NW) % MT);
    }
  }
  if (XNORM) sk_ssq_ask<NW, MT>(sq, M, nrm, sq_row);
  for (int i = 0; i < n_it; ++i) {
    bf16x8 wnow[NWT][2];   // (wl 1, 2) this pair's operands of W, which the next pair's loads are about to replace
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (t < NWT && wl != 0) {
        wnow[t][0] = held[t][0];
        wnow[t][1] = held[t][1];
      } else {
        *(bf16x8*)(stage + t * 2048 + (t < NWT ? putw0 : put0)) = held[t][0];
        *(bf16x8*)(stage + t * 2048 + (t < NWT ? putw1 : put1)) = held[t][1];
      }
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
          const bf16x8 wf = wl != 0 ? wnow[g * NG + h][s] : *(const bf16x8*)(stage + (g * NG + h) * 2048 + get);
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
#ifdef SK_STAMPS
  asm volatile("s_nop 0" :: "v"(acc[0][0][0][0]));
  SK_STAMP(4);
#endif
  if (XNORM) sk_ssq_sum<NW, MT>(sm_ssq, sq, M, nrm, sq_row, acc[0][0][0][0]);   // (read after the barrier before the first strip's end)
  SK_STAMP(5);
  // All strips of the block end together: every wave's partial tiles go to shared memory, tile t is summed in wave
  // order by wave t % NW, and wave g * MT + mt finishes token tile mt of strip g (three barriers a block, not three a strip).
  __syncthreads();   // the staged lines are free
#pragma unroll
  for (int g = 0; g < NS; ++g)
#pragma unroll
    for (int h = 0; h < NG; ++h)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) red[wave][(g * NG + h) * MT + mt][lane] = acc[g][h][mt];
  __syncthreads();
  SK_STAMP(6);
  for (int t = wave; t < NTILES; t += NW) {
    f32x4 v = red[0][t][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) v += red[w][t][lane];
    red[0][t][lane] = v;   // only this thread touches red[*][t][lane] before the barrier
  }
  __syncthreads();
  SK_STAMP(7);
#pragma unroll
  for (int e = 0; e < ENDS; ++e) {
    const int end_g = (wave + e * NW) / MT, end_mt = (wave + e * NW) % MT;
    if (wave + e * NW < NS * MT && strip0 + end_g < n_strips) {
      const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
      sk_end_tile<MT, NW, EPI, TC, XNORM, false>(red[0][end_g * NG * MT + end_mt][lane],
                                                 (EPI == SK_GATED) ? red[0][(end_g * NG + 1) * MT + end_mt][lane] : zero4, end_mt,
                                                 sm_ssq, strip0 + end_g, end_hd[e], end_sub[e], end_rot[e], out, M, N, K, ldc, nrm,
                                                 nullptr, rp, nx, pre[e]);
    }
  }
  SK_STAMP(9); SK_STAMP(15);
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
  int wl = 0;                 // (kernel of whole lines) W points at: 0 the stored rows, 1 the operands' order, 2 the packed strips of 8
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
    if constexpr (NW == 16 && KS >= 8)                                                                            \
      gemm_skinny_resident_kernel<MT, NW, KS, EPI, TC, XNORM, SSQ, 2>                                             \
          <<<dim3(resident_blocks(n_strips, NW)), dim3(NW * 64), 0, a.stream>>>(                                  \
              a.A, (const bf16_t*)a.W, (TC*)a.C, a.M, a.N, a.K, a.lda, a.ldw, a.ldc, a.nrm, a.ssq_out, a.nx, a.rp, n_strips, \
              (const bf16_t*)a.Wt);                                                                               \
    else if (a.Wt)                                                                                                \
      gemm_skinny_resident_kernel<MT, NW, KS, EPI, TC, XNORM, SSQ, 1>                                             \
          <<<dim3(resident_blocks(n_strips, NW)), dim3(NW * 64), 0, a.stream>>>(                                  \
              a.A, (const bf16_t*)a.W, (TC*)a.C, a.M, a.N, a.K, a.lda, a.ldw, a.ldc, a.nrm, a.ssq_out, a.nx, a.rp, n_strips, \
              (const bf16_t*)a.Wt);                                                                               \
    else                                                                                                          \
      gemm_skinny_resident_kernel<MT, NW, KS, EPI, TC, XNORM, SSQ, 0>                                             \
          <<<dim3(resident_blocks(n_strips, NW)), dim3(NW * 64), 0, a.stream>>>(                                  \
              a.A, (const bf16_t*)a.W, (TC*)a.C, a.M, a.N, a.K, a.lda, a.ldw, a.ldc, a.nrm, a.ssq_out, a.nx, a.rp, n_strips, \
              (const bf16_t*)nullptr);                                                                            \
    GL3_LAUNCH_CHECK();                                                                                           \
    return 0;                                                                                                     \
  } while (0)
  if constexpr (MT == 1 && !XNORM && (EPI == SK_STORE || EPI == SK_ADD)) {
    if (a.strip_rows == 8) {
      // strips of 8 rows: twice the blocks, each with half the rows to stream; with at most 8 rows of A
      // the tile's other half takes the next 32 k
      if (a.M <= 8 && a.Wt8 && a.lda < (1L << 24) && a.K < (1 << 24))   // (32-bit byte offsets inside a strip and inside A)
        gemm_skinny_pack_kernel<16, EPI, TC, SSQ><<<dim3((a.N + 7) / 8), dim3(16 * 64), 0, a.stream>>>(
            (const bf16_t*)a.A, (const bf16_t*)a.Wt8, (TC*)a.C, a.M, a.N, a.K, (int)a.lda, a.ldc, a.ssq_out, a.nx, a.a_packed);
      else if (a.M <= 8)
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
  if constexpr (MT == 1 && XNORM && !SSQ) {
    // a decode step's products with a folded norm over the copy of W: the kernel with the short prologue
    if (a.resident && a.Wt && a.lda < (1L << 24) && a.K < (1 << 24) && (long)steps * 1024 < (1L << 31)) {
#ifndef SK_DEC_NW
#define SK_DEC_NW 16
#endif
#define DEC(KS)                                                                                                  \
  do {                                                                                                           \
    gemm_skinny_decode_kernel<SK_DEC_NW, KS * 16 / SK_DEC_NW, EPI, TC><<<dim3(resident_blocks(n_strips, SK_DEC_NW)), dim3(SK_DEC_NW * 64), 0, a.stream>>>( \
        (const bf16_t*)a.A, (const bf16_t*)a.Wt, (TC*)a.C, a.M, a.N, a.K, (int)a.lda, a.ldc, a.nrm, a.nx, a.rp, n_strips); \
    GL3_LAUNCH_CHECK();                                                                                          \
    return 0;                                                                                                    \
  } while (0)
      if (steps <= 64) DEC(4);
      if constexpr (EPI == SK_STORE || EPI == SK_QKV) {
        if (steps <= 96) DEC(6);   // (the QKV product of the 3B layers, K = 3,072: 13.8 us on the streaming kernel, 11.1 us here)
      }
      if constexpr (EPI == SK_STORE) {   // (with the rotation's operands beside 8 k-steps a wave the registers spill: K = 4,096, 17.0 -> 18.6 us)
        if (steps <= 128) DEC(8);
      }
#undef DEC
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
    // 16 waves a strip where their partial tiles fit, so that a strip's rows are asked for at once; with three and
    // four token tiles only for the plain store (the head of 33 to 64 rows: 122.5 -> 115.5 us at 64), whose registers
    // hold them; a folded norm, the sums of squares or the rotation's operands beside them spill
    if constexpr (NG * MT <= 2 || (EPI == SK_STORE && !XNORM && !SSQ && MT <= 4)) {
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
#define SK_WIDE(WL)                                                                                               \
  gemm_skinny_wide_kernel<MT, NS, NW, EPI, TC, XNORM, WL>                                                         \
      <<<dim3((n_strips + NS - 1) / NS, slices), dim3(NW * 64), 0, a.stream>>>(                                   \
          (const bf16_t*)a.A, (const bf16_t*)a.W, (TC*)a.C, a.M, a.N, a.K, a.lda, a.ldw, a.ldc, slice_stride, per_slice, \
          a.rp, a.nx, a.nrm)
  if (a.wl == 0) SK_WIDE(0);
  else if (a.wl == 1) SK_WIDE(1);
  else {
    // the packed strips of 8 rows: the copies of the output and down projections
    if constexpr ((EPI == SK_STORE || EPI == SK_ADD) && !XNORM) SK_WIDE(2);
    else GL3_REQUIRE(false, "gl3_gemm_skinny_wide: W in packed strips of 8 is read by the store and add epilogues (epilogue %d)", EPI);
  }
#undef SK_WIDE
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
                                    float eps, int pack_out, int w_order, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (check_common("gl3_gemm_skinny_wide", A, W, C, M, N, K, lda, ldw, 0)) return -1;
  // w_order: 0: W holds the rows as they are stored. 1: W is the copy in the matrix operands' order (lib.tile_weight,
  // rows in order; gated: the gate strips, then the up strips). 2: the copy in packed strips of 8 rows (lib.tile_weight8).
  {
    const long w_rows = epilogue == SK_GATED ? 2L * N : N;
    GL3_REQUIRE(w_order >= 0 && w_order <= 2 && (w_order != 1 || (N % 16 == 0 && w_rows * ((K + 31) / 32 * 64) < (1L << 31))) &&
                    (w_order != 2 || (N % 8 == 0 && epilogue != SK_GATED && (long)N * ((K + 63) / 64 * 128) < (1L << 31))),
                "gl3_gemm_skinny_wide: W in order %d with N=%d, K=%d, epilogue %d", w_order, N, K, epilogue);
  }
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
  a.wl = w_order;
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
                                  const void* w_tiled, const int* token_pages, const float* token_rot, int w_once,
                                  hipStream_t stream) {
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
  GL3_REQUIRE(!token_pages || !cos_tab || token_rot, "gl3_qkv_rope_cache: the tokens' pages come with their rows of cos and sin");
  const SkRope rp = {positions, seq_of_token, block_table, table_stride, cos_tab, sin_tab, (bf16_t*)k_cache,
                     (bf16_t*)v_cache, n_heads, n_kv, head_dim, adjacent, page_size, token_pages, token_rot};
  SkCall a = {a_rows, Wqkv, q_out, M, N, K, lda, ldw, ldq, nrm, nullptr, rp, stream, waves == 0};
  GL3_REQUIRE(!w_tiled || (uintptr_t)w_tiled % 16 == 0, "gl3_qkv_rope_cache: the copy of W must be 16-byte aligned");
  a.Wt = w_tiled;   // (its strips hold the rows that sk_strip_row names: for half-split pairing 8 rows and the 8 half a head further)
  // w_once: the stored order is gone, Wqkv is that copy: the kernels of few rows read it as before, the kernel of
  // whole lines reads it in its own order
  GL3_REQUIRE(!w_once || (w_tiled && N % 16 == 0 && (long)N * ((K + 31) / 32 * 64) < (1L << 31)),
              "gl3_qkv_rope_cache: weights in the operands' order alone need that copy (N=%d, K=%d)", N, K);
  if (w_once) { a.W = w_tiled; a.wl = 1; }
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
  // a folded norm's product of one token tile over a K too long for the kernel that keeps its operands in registers:
  // whole lines, one strip a block, of which a CU holds several (so that more strips than CUs do not wait for a
  // second round)
  if (ssq && waves == 0 && M <= 16 && K > 3072 && wide_addressable(M, N, K, lda, ldw))
    return launch_wide<1, 1, SK_QKV, bf16_t, true>(a, 1, 0);
  if (!ssq) return pick_mt<SK_QKV, bf16_t, false, false>(pick_waves(waves, N, K), a);
  return pick_mt<SK_QKV, bf16_t, true, false>(pick_waves(waves, N, K), a);
}

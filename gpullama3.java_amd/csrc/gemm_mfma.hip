// C[M,N] = A[M,K] . W[N,K]^T in bfloat16 on the matrix cores for many rows of A: the
// products of a prefill step. 32-bit accumulation; W is row-major [out, in]
// (J/core/model/tensor/FloatTensor.java:98-100).
//
// A block is WM x WN waves; each wave owns 64 x 64 (or 32 x 64) of the block's tile of C as
// 2 x 2 (1 x 2) tiles of the 32x32x16 instruction: sixteen waves on 256 x 256 for large products,
// eight waves on 128 x 128 otherwise. For the gated epilogue a W tile holds the gate rows of
// half as many output columns and the matching up rows. K advances in steps of 64 through two
// buffers in shared memory: while a step's products run out of one, the next step's operands go
// from registers into the other and the step after that travels from memory to registers; one
// barrier a step. Rows in shared memory are padded by 16 bytes so that the 32 lanes that read one
// column of 16-byte operands hit different banks.
// Blocks are numbered so that each XCD (whose second-level cache is its own) works on a
// contiguous range of tiles, ordered so that the tiles it holds at one time form a rectangle
// and share their panels of A and of W.
//
// Epilogues as in gemm_generic.hip: store, add into a float matrix, gated.
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { MF_STORE = 0, MF_ADD = 1, MF_GATED = 2 };

#define MF_BK 64
#define MF_LD (MF_BK + 8)   // padded row, in elements

// WM x WN waves; a wave owns (32*TM) x 64 of the tile.
template <int EPI, typename TC, int TM, int WM, int WN, int WT = 0>
__global__ __launch_bounds__(64 * WM * WN) void gemm_mfma_kernel(const bf16_t* __restrict__ A,
                                                                  const bf16_t* __restrict__ W, TC* __restrict__ C,
                                                                  int M, int N, int K, long lda, long ldw, long ldc,
                                                                  int tiles_m, int tiles_n, int group_m, int k_per_slice,
                                                                  float* __restrict__ P, long p_stride, long ldp,
                                                                  const float* __restrict__ bias, int act, int w_steps,
                                                                  const int* __restrict__ w_pos) {
  constexpr int NT = 64 * WM * WN;                       // threads
  constexpr int BM = 32 * TM * WM;                       // rows of a block
  constexpr int BN = 64 * WN;                            // rows of W of a block
  constexpr int NCOLS = (EPI == MF_GATED) ? BN / 2 : BN; // output columns of a block
  constexpr int NA = BM * 8 / NT;                        // 16-byte chunks of A per thread and k-step
  constexpr int NWC = BN * 8 / NT;                       // and of W
  static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile does not divide over the threads");
  __shared__ __attribute__((aligned(16))) bf16_t As[2][BM][MF_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][BN][MF_LD];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave / WN, wn = wave % WN;
  const int lr = lane & 31, lh = lane >> 5;

  // block -> tile: 8 XCDs take turns on consecutive block ids; give each a contiguous range
  const int n_tiles = tiles_m * tiles_n;
  const int per_xcd = (n_tiles + 7) / 8;
  const int tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (tile >= n_tiles) return;
  // the tiles in order: bands of group_m row tiles; inside a band column after column, the band's row
  // tiles of a column one after the other. The tiles that an XCD works on at one time are then a
  // rectangle of group_m row tiles by a few column tiles, which share their rows of A and of W.
  const int band = tile / (group_m * tiles_n), in_band = tile % (group_m * tiles_n);
  const int band_rows = min(group_m, tiles_m - band * group_m);
  const int m0 = (band * group_m + in_band % band_rows) * BM;
  const int n0 = (in_band / band_rows) * NCOLS;

  // global -> register staging in chunks of 16 bytes. An address is a base that the whole block
  // shares (it lives in scalar registers and takes the k-step) plus a 32-bit offset of the thread
  // inside the tile, and every load is unconditional (rows and columns beyond the matrix are
  // clamped to its last ones and their values dropped): no branch around a load, whose registers
  // the compiler would then wait for at once.
  // WT 1: W is the copy in the matrix operands' order alone ([strip of 16 rows][k-step of 32][lane][8], w_steps
  // k-steps a strip, gl3_operand_offset; w_pos, may be null: each row's place in a copy whose strips hold the rows
  // in another order). WT 2: the copy in packed strips of 8 rows (gl3_packed_offset, w_steps steps of 64). A
  // thread's 16 bytes are still 8 consecutive k of one row, only at another place, and go to the same place in
  // shared memory.
  const bf16_t* a_tile = A + (long)m0 * lda;
  const bf16_t* w_tile[2];
  w_tile[0] = WT ? W : W + (long)n0 * ldw;
  w_tile[1] = WT ? W : (EPI == MF_GATED) ? W + ((long)N + n0) * ldw : w_tile[0];
  static_assert(EPI != MF_GATED || (NWC % 2 == 0 && (NT / 8) * (NWC / 2) == BN / 2),
                "gate rows and up rows must fall to different loads of a thread");
  unsigned aoff[NA], woff[NWC];
  int arow_s[NA], wrow_s[NWC], wcol_s[NWC];
  const int scol = (tid & 7) * 8;
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    arow_s[i] = (tid + NT * i) >> 3;
    aoff[i] = (unsigned)(min(m0 + arow_s[i], M - 1) - m0) * (unsigned)lda;
  }
#pragma unroll
  for (int i = 0; i < NWC; ++i) {
    int r = (tid + NT * i) >> 3, c = tid & 7;
    if (WT) {
      // Which 16 bytes of the tile a thread brings is free (they go to their own place in shared memory). In a copy's
      // order 8 rows of a strip at one block of 8 k are a 128-byte line. With the stored order's assignment (eight
      // neighbouring threads: the eight pieces of one row's 64 k) eight threads would touch eight lines, 16 bytes of
      // each, which a CU's first-level cache takes at a third of the rate of whole lines (the products of 2,048 rows
      // were 13 to 20% slower that way). So eight neighbouring threads take one whole line, and a wave the same
      // line of 8 different strips: lane l the row l % 8 of strip l / 8 of its group.
      const int idx = (tid >> 6) * NWC + i, l = tid & 63;
      if (WT == 1) {   // [strip of 16][k-step of 32][k block q][row][8]: 16 lines a strip and step of 64 k
        const int combo = idx & 15;
        r = ((idx >> 4) * 8 + (l >> 3)) * 16 + (combo & 1) * 8 + (l & 7);
        c = (combo >> 3) * 4 + ((combo >> 1) & 3);
      } else {         // [strip of 8][step of 64 k][k block q][half][row][8]: 8 lines a strip and step
        const int combo = idx & 7;
        r = ((idx >> 3) * 8 + (l >> 3)) * 8 + (l & 7);
        c = (combo & 1) * 4 + (combo >> 1);
      }
    }
    wrow_s[i] = r;
    wcol_s[i] = c * 8;
    // (gated: the tile's second half of rows are the up rows of the same columns; in a copy's order which half a
    // load falls into goes by its row, not by its number)
    const bool up = EPI == MF_GATED && (WT ? r >= BN / 2 : i >= NWC / 2);
    const int rel = up ? r - BN / 2 : r;
    const int row = min(n0 + rel, N - 1);
    const int wrow = row + (up ? N : 0);
    // (WT: K is a multiple of 64, so a thread's column inside a k-step of 64 is at the same place of every step)
    woff[i] = WT == 1   ? (unsigned)gl3_operand_offset(w_pos ? w_pos[wrow] : wrow, c * 8, w_steps)
              : WT == 2 ? (unsigned)gl3_packed_offset(wrow, c * 8, w_steps)
                        : (unsigned)(row - n0) * (unsigned)ldw;
  }
  // K in slices (blockIdx.y): slice 0 ends in the epilogue proper, the others store their sums
  // as floats into P[slice - 1], for the reader to add up in slice order
  const int slice = blockIdx.y;
  const int k_begin = slice * k_per_slice;
  K = min(K, k_begin + k_per_slice);
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 ra[NA], rw[NWC];
  bool r_ok = false;                                   // whether the registers hold columns inside K
  auto fetch = [&](int k0) {
    const int kf = min(k0, K - 8);                     // the step after the last one reads the last again
    r_ok = k0 + scol < K;
    const unsigned col = (unsigned)min(scol, K - 8 - kf);
    const bf16_t* ak = a_tile + kf;
#pragma unroll
    for (int i = 0; i < NA; ++i) ra[i] = *(const bf16x8*)(ak + (aoff[i] + col));
    if (WT) {
      // a k-step of 64 lies 2 KB (the operands' order: two k-steps of 32) or 1 KB (the packed strips of 8) further in
      // every strip: the same step for all threads, whose offsets stay what they are
      const bf16_t* wk = w_tile[0] + (long)(min(k0, K - 64) >> 6) * (WT == 1 ? 1024 : 512);   // (the step after the last reads the last again)
#pragma unroll
      for (int i = 0; i < NWC; ++i) rw[i] = *(const bf16x8*)(wk + woff[i]);
    } else {
#pragma unroll
      for (int i = 0; i < NWC; ++i) {
        const bf16_t* wk = w_tile[(EPI == MF_GATED && i >= NWC / 2) ? 1 : 0] + kf;
        rw[i] = *(const bf16x8*)(wk + (woff[i] + col));
      }
    }
  };
  fetch(k_begin);

  f32x16 acc[TM][2];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int jn = 0; jn < 2; ++jn)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][jn][v] = 0.f;

  const int arow = wm * 32 * TM + lr;
  const int wrow0 = (EPI == MF_GATED) ? wn * 32 + lr : wn * 64 + lr;
  const int wrow1 = (EPI == MF_GATED) ? BN / 2 + wn * 32 + lr : wn * 64 + 32 + lr;

  // registers -> shared memory; a step that reaches beyond K drops the columns from K on
  auto store = [&](int buf, int k0) {
    if (k0 + MF_BK <= K) {   // a whole step (the same for the whole block): nothing to drop
#pragma unroll
      for (int i = 0; i < NA; ++i) *(bf16x8*)&As[buf][arow_s[i]][scol] = ra[i];
#pragma unroll
      for (int i = 0; i < NWC; ++i) *(bf16x8*)&Ws[buf][wrow_s[i]][WT ? wcol_s[i] : scol] = rw[i];
    } else {
#pragma unroll
      for (int i = 0; i < NA; ++i) *(bf16x8*)&As[buf][arow_s[i]][scol] = r_ok ? ra[i] : zero;
#pragma unroll
      for (int i = 0; i < NWC; ++i) *(bf16x8*)&Ws[buf][wrow_s[i]][WT ? wcol_s[i] : scol] = r_ok ? rw[i] : zero;
    }
  };
  auto products = [&](int buf, int kk) {
    const int kc = kk * 16 + lh * 8;
    const bf16x8 b0 = *(const bf16x8*)&Ws[buf][wrow0][kc];
    const bf16x8 b1 = *(const bf16x8*)&Ws[buf][wrow1][kc];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const bf16x8 a = *(const bf16x8*)&As[buf][arow + 32 * tm][kc];
      acc[tm][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, acc[tm][0], 0, 0, 0);
      acc[tm][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, acc[tm][1], 0, 0, 0);
    }
  };
  // Two buffers in shared memory: while a step's products run out of one, the next step's operands
  // (in registers since the step before) are written to the other and the step after that is asked
  // for; one barrier a step.
  store(0, k_begin);
  fetch(k_begin + MF_BK);
  __syncthreads();
  int buf = 0;
  for (int k0 = k_begin; k0 < K; k0 += MF_BK, buf ^= 1) {
#pragma unroll
    for (int kk = 0; kk < MF_BK / 16; ++kk) {
      products(buf, kk);
      if (kk == 0) {
        // behind the first products (which cover the wait for the registers and the address
        // arithmetic); the scheduler may not move the loads or the writes across the fences
        __builtin_amdgcn_sched_barrier(0);
        if (k0 + MF_BK < K) store(buf ^ 1, k0 + MF_BK);
        fetch(k0 + 2 * MF_BK);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();
  }

  // lane holds C[row(v)][col]: row(v) = 8*(v/4) + 4*(lane/32) + v%4 inside a 32x32 tile, col = lane%32.
  // Whole tiles (all but the matrix's last row and column of tiles) store without a test per element.
  auto finish = [&](auto checked_t) {
    constexpr bool CHECKED = decltype(checked_t)::value;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * 32 * TM + tm * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
        if (CHECKED && m >= M) continue;
        if (slice > 0) {
#pragma unroll
          for (int tn = 0; tn < 2; ++tn) {
            const int n = n0 + wn * 64 + tn * 32 + lr;
            if (!CHECKED || n < N) P[(long)(slice - 1) * p_stride + (long)m * ldp + n] = acc[tm][tn][v];
          }
          continue;
        }
        if (EPI == MF_GATED) {
          const int n = n0 + wn * 32 + lr;
          if (!CHECKED || n < N) {
            float g = acc[tm][0][v], u = acc[tm][1][v];
            if (bias) { g += bias[n]; u += bias[N + n]; }
            C[(long)m * ldc + n] = from_f32<TC>(gl3_activation<true>(g, act) * u);
          }
        } else {
#pragma unroll
          for (int tn = 0; tn < 2; ++tn) {
            const int n = n0 + wn * 64 + tn * 32 + lr;
            if (!CHECKED || n < N) {
              TC* c = C + (long)m * ldc + n;
              const float s = acc[tm][tn][v] + (bias ? bias[n] : 0.f);
              if (EPI == MF_ADD) *c = from_f32<TC>(to_f32<TC>(*c) + s);
              else *c = from_f32<TC>(s);
            }
          }
        }
      }
    }
  };
  if (m0 + BM <= M && n0 + NCOLS <= N) finish(std::false_type{});
  else finish(std::true_type{});
}

template <int EPI, typename TC, int TM, int WM, int WN, int WT = 0>
static int launch_shape(const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw, long ldc,
                        int slices, float* P, long p_stride, long ldp, const float* bias, int act, int w_steps,
                        const int* w_pos, hipStream_t stream) {
  const int bm = 32 * TM * WM;
  const int ncols = (EPI == MF_GATED) ? 32 * WN : 64 * WN;
  const int tiles_n = (N + ncols - 1) / ncols;
  const int tiles_m = (M + bm - 1) / bm;
  const long n_tiles = (long)tiles_m * tiles_n;
  const long blocks = ((n_tiles + 7) / 8) * 8;
  GL3_REQUIRE(blocks < (1L << 31), "gl3_gemm_mfma: too many tiles");
  const int k_per_slice = ((K + MF_BK - 1) / MF_BK + slices - 1) / slices * MF_BK;
  // 32 tiles of 256 x 256 (64 of 128 x 128) run on an XCD at a time: bands of 4 (8) row tiles make
  // them a rectangle of 4 x 8 (8 x 8), which asks memory for a third of the bytes that one column of
  // 32 row tiles does (3 to 5% of the time of the large products)
  const int group_m = tiles_m < (bm == 256 ? 4 : 8) ? tiles_m : (bm == 256 ? 4 : 8);
  gemm_mfma_kernel<EPI, TC, TM, WM, WN, WT><<<dim3((unsigned)blocks, slices), dim3(64 * WM * WN), 0, stream>>>(
      (const bf16_t*)A, (const bf16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, tiles_m, tiles_n, group_m, k_per_slice, P,
      p_stride, ldp, bias, act, w_steps, w_pos);
  GL3_LAUNCH_CHECK();
  return 0;
}

// The tile the library takes where the caller names none: 1 (128 x 128), 2 (256 x 256) or 5 (128 rows x 256).
// 256 x 256 tiles of sixteen waves, one block a CU, have half the operand traffic per product, and
// that traffic is what bounds the large products; of the 128 x 128 tiles of eight waves two fit a CU and
// overlap each other's waits. A step of 64 columns takes a chip full of the large tiles 1.7 us and a chip
// full of the small ones (twice as many blocks, a quarter of the work each) 1.05 us, and the blocks need
// rounds on the chip: the tile whose rounds take less time is chosen (240 large tiles are one round
// where 960 small ones are two; 276 large ones are two where 1,104 small ones are three).
// A third tile, 128 rows x 256 of sixteen waves of 32 x 64, is for the products in between: more tiles of 128 x 128
// than one for every CU, but not enough work to fill the chip with the large tiles (2,048 rows of the 1B layers'
// QKV product, 384 tiles of 128 x 128 or 192 of 128 x 256: 45 -> 40 us); a step of it takes a full chip about 0.95 us.
// Tiles of 128 x 128 that are at most one a CU run faster than two that share one (0.8 of the time a step).
static int choose_shape(int M, int N, int slices, bool gated) {
  const long small_n = gated ? (N + 63) / 64 : (N + 127) / 128;
  const long big_n = gated ? (N + 127) / 128 : (N + 255) / 256;
  const long small_tiles = (long)((M + 127) / 128) * small_n * slices, wide_tiles = (long)((M + 127) / 128) * big_n * slices;
  const long big_tiles = (long)((M + 255) / 256) * big_n * slices;
  // rounds on the chip, in thousandths: whole rounds, and a last, partly empty one that costs half a round and
  // half of the share of the places it fills (a chip half full works through its blocks faster, not twice as fast)
  auto rounds = [](long tiles, long places) { return tiles / places * 1000 + (tiles % places ? 500 + tiles % places * 500 / places : 0); };
  const long small_cost = rounds(small_tiles, 512) * (small_tiles <= 256 ? 84 : 105), big_cost = rounds(big_tiles, 256) * 170;
  const long wide_cost = rounds(wide_tiles, 256) * (wide_tiles <= 128 ? 119 : 95);
  if (wide_cost < small_cost && wide_cost < big_cost && slices == 1) return 5;
  return big_cost < small_cost ? 2 : 1;
}

template <int EPI, typename TC>
static int launch_mfma(const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw, long ldc,
                       int slices, float* P, long p_stride, long ldp, const float* bias, int act, int shape, int w_order,
                       const int* w_pos, hipStream_t stream) {
  const int w_steps = w_order == 1 ? (K + 31) / 32 : w_order == 2 ? (K + 63) / 64 : 0;
  if (shape == 0) shape = choose_shape(M, N, slices, EPI == MF_GATED);
#define MF_ARGS A, W, C, M, N, K, lda, ldw, ldc, slices, P, p_stride, ldp, bias, act, w_steps, w_pos, stream
  if (w_order) {
    // W is one of its copies in the matrix cores' order (a weight that is held once): the three tiles that the library
    // chooses between
    GL3_REQUIRE(shape == 1 || shape == 2 || shape == 5, "gl3_gemm_mfma: tile shape %d does not read W in a copy's order", shape);
    if (w_order == 1)
      return shape == 1 ? launch_shape<EPI, TC, 1, 4, 2, 1>(MF_ARGS)
             : shape == 2 ? launch_shape<EPI, TC, 2, 4, 4, 1>(MF_ARGS) : launch_shape<EPI, TC, 1, 4, 4, 1>(MF_ARGS);
    if constexpr (EPI != MF_GATED) {
      return shape == 1 ? launch_shape<EPI, TC, 1, 4, 2, 2>(MF_ARGS)
             : shape == 2 ? launch_shape<EPI, TC, 2, 4, 4, 2>(MF_ARGS) : launch_shape<EPI, TC, 1, 4, 4, 2>(MF_ARGS);
    } else {
      GL3_REQUIRE(false, "gl3_gemm_mfma: the gated epilogue reads the copy in the operands' order, not the packed strips of 8 (order %d)", w_order);
    }
  }
  if (shape == 1) return launch_shape<EPI, TC, 1, 4, 2>(MF_ARGS);
  if (shape == 2) return launch_shape<EPI, TC, 2, 4, 4>(MF_ARGS);
  if (shape == 3) return launch_shape<EPI, TC, 4, 2, 4>(MF_ARGS);
  if (shape == 4) return launch_shape<EPI, TC, 2, 4, 2>(MF_ARGS);
  return launch_shape<EPI, TC, 1, 4, 4>(MF_ARGS);
#undef MF_ARGS
}

// N counts output columns: for the gated epilogue W has 2N rows (gate, then up).
// slices > 1 (not with the gated epilogue): K is cut into that many slices; the first ends in the
// epilogue into C, slice s > 0 stores its sums into P[s - 1] ([slices - 1][M][ldp] floats,
// p_stride elements apart), which the caller adds to C in that order.
// bias (may be null; not with slices): N floats (gated: 2N). act: the gated epilogue's activation.
// shape: 0 lets the library choose the tile; 1: 128 x 128, eight waves; 2: 256 x 256, sixteen waves of
// 64 x 64; 3: 256 x 256, eight waves of 128 x 64; 4: 256 rows x 128, eight waves of 64 x 64; 5: 128 rows x 256,
// sixteen waves of 32 x 64.
// w_order, w_pos: how W lies (see below): as stored, or one of its copies in the matrix cores' order alone.
extern "C" int gl3_gemm_mfma(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, long lda, long ldw,
                             long ldc, int epilogue, int slices, float* P, long p_stride, long ldp, const float* bias,
                             int act, int shape, int w_order, const int* w_pos, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  GL3_REQUIRE(A && W && C && M > 0 && N > 0 && K > 0, "gl3_gemm_mfma: bad arguments (M=%d N=%d K=%d)", M, N, K);
  GL3_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gl3_gemm_mfma: K=%d, lda=%ld, ldw=%ld must be multiples of 8",
              K, lda, ldw);
  GL3_REQUIRE(lda > 0 && ldw > 0 && lda < (1L << 22) && ldw < (1L << 22),
              "gl3_gemm_mfma: lda=%ld, ldw=%ld: rows of 2^22 elements or more are not built (32-bit offsets in a tile)",
              lda, ldw);
  GL3_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "gl3_gemm_mfma: operands must be 16-byte aligned");
  GL3_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gl3_gemm_mfma: leading dimensions too small");
  GL3_REQUIRE(epilogue >= 0 && epilogue <= 2, "gl3_gemm_mfma: unknown epilogue %d", epilogue);
  GL3_REQUIRE(epilogue != MF_ADD || c_dtype == GL3_F32, "gl3_gemm_mfma: the add epilogue needs a float output");
  GL3_REQUIRE(slices >= 1 && slices <= 64 && slices <= (K + MF_BK - 1) / MF_BK, "gl3_gemm_mfma: %d slices of K=%d",
              slices, K);
  GL3_REQUIRE(slices == 1 || (epilogue != MF_GATED && P && ldp >= N && p_stride >= (long)(M - 1) * ldp + N),
              "gl3_gemm_mfma: slices need a buffer for their sums and another epilogue than the gated one");
  GL3_REQUIRE(!bias || slices == 1, "gl3_gemm_mfma: a bias goes with one slice of K");
  GL3_REQUIRE(act == GL3_ACT_SILU || act == GL3_ACT_GELU_TANH, "gl3_gemm_mfma: unknown activation %d", act);
  GL3_REQUIRE(shape >= 0 && shape <= 5, "gl3_gemm_mfma: unknown tile shape %d", shape);
  // w_order: 0: W holds the rows as stored. 1: W is the copy in the matrix operands' order (lib.tile_weight), w_pos (may be
  // null) naming each row's place in it. 2: the copy in packed strips of 8 rows (lib.tile_weight8).
  {
    const long w_rows = epilogue == MF_GATED ? 2L * N : (long)N;
    GL3_REQUIRE(w_order >= 0 && w_order <= 2 && (w_order == 0 || (K % 64 == 0 && (long)w_rows * K < (1L << 32))) &&
                    (w_order != 1 || (w_rows % 16 == 0 && N % 16 == 0)) && (w_order != 2 || w_rows % 8 == 0) && (w_order == 1 || !w_pos),
                "gl3_gemm_mfma: W in order %d with K=%d (a copy's order is read over whole steps of 64), N=%d", w_order, K, N);
  }
#define ARGS A, W, C, M, N, K, lda, ldw, ldc, slices, P, p_stride, ldp, bias, act, shape, w_order, w_pos, stream
  if (c_dtype == GL3_F32) {
    if (epilogue == MF_STORE) return launch_mfma<MF_STORE, float>(ARGS);
    if (epilogue == MF_ADD) return launch_mfma<MF_ADD, float>(ARGS);
    return launch_mfma<MF_GATED, float>(ARGS);
  } else if (c_dtype == GL3_BF16) {
    if (epilogue == MF_STORE) return launch_mfma<MF_STORE, bf16_t>(ARGS);
    if (epilogue == MF_GATED) return launch_mfma<MF_GATED, bf16_t>(ARGS);
  }
#undef ARGS
  GL3_REQUIRE(false, "gl3_gemm_mfma: unsupported output dtype %d for epilogue %d", c_dtype, epilogue);
  return 0;
}

// C[M,N] = A[M,K] . W[N,K]^T in bfloat16 on the matrix cores for many rows of A: the
// products of a prefill step. 32-bit accumulation; W is row-major [out, in]
// (J/core/model/tensor/FloatTensor.java:98-100).
//
// A block of four waves computes a 128 x 128 tile of C (128 x 64 for the gated epilogue,
// whose W tile holds 64 gate rows and the 64 matching up rows; 64 x 128 when the matrix
// would otherwise give fewer tiles than two per CU). K advances in steps of
// 64: the next step's operands travel from memory to registers while the matrix cores
// work on the current step out of shared memory. Each wave owns 64 x 64 (or 32 x 64) of
// the tile as 2 x 2 (1 x 2) tiles of the 32x32x16 instruction. Rows in shared memory are
// padded by 16 bytes so that the 32 lanes that read one column of 16-byte operands hit
// different banks.
// Blocks are numbered so that each XCD (whose second-level cache is its own) works on a
// contiguous range of tiles, neighbouring tiles sharing their panel of W.
//
// Epilogues as in gemm_generic.hip: store, add into a float matrix, gated.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { MF_STORE = 0, MF_ADD = 1, MF_GATED = 2 };

#define MF_BM 128
#define MF_BN 128
#define MF_BK 64
#define MF_LD (MF_BK + 8)   // padded row, in elements

template <int EPI, typename TC, int TM>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                        TC* __restrict__ C, int M, int N, int K, long lda, long ldw,
                                                        long ldc, int tiles_m, int tiles_n) {
  constexpr int NCOLS = (EPI == MF_GATED) ? 64 : 128;   // output columns of a block
  constexpr int BM = 64 * TM;                            // rows of a block
  constexpr int NA = BM / 32;                            // 16-byte chunks of A per thread and k-step
  __shared__ __attribute__((aligned(16))) bf16_t As[BM][MF_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[MF_BN][MF_LD];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 31, lh = lane >> 5;

  // block -> tile: 8 XCDs take turns on consecutive block ids; give each a contiguous range
  const int n_tiles = tiles_m * tiles_n;
  const int per_xcd = (n_tiles + 7) / 8;
  const int tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (tile >= n_tiles) return;
  const int m0 = (tile % tiles_m) * BM;
  const int n0 = (tile / tiles_m) * NCOLS;

  // global -> register staging: chunks of 16 bytes, NA of A and 4 of W per thread
  const bf16_t* ap[NA];
  const bf16_t* wp[4];
  int srow[4], scol[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + 256 * i;
    srow[i] = c >> 3;
    scol[i] = (c & 7) * 8;
    if (i < NA) ap[i] = A + (long)min(m0 + srow[i], M - 1) * lda + scol[i];
    int wr;
    if (EPI == MF_GATED) wr = srow[i] < 64 ? min(n0 + srow[i], N - 1) : N + min(n0 + srow[i] - 64, N - 1);
    else wr = min(n0 + srow[i], N - 1);
    wp[i] = W + (long)wr * ldw + scol[i];
  }
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 ra[NA], rw[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bool ok = scol[i] < K;
    if (i < NA) ra[i] = ok ? *(const bf16x8*)ap[i] : zero;
    rw[i] = ok ? *(const bf16x8*)wp[i] : zero;
  }

  f32x16 acc[TM][2];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int jn = 0; jn < 2; ++jn)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][jn][v] = 0.f;

  const int arow = wm * 32 * TM + lr;
  const int wrow0 = (EPI == MF_GATED) ? wn * 32 + lr : wn * 64 + lr;
  const int wrow1 = (EPI == MF_GATED) ? 64 + wn * 32 + lr : wn * 64 + 32 + lr;

  for (int k0 = 0; k0 < K; k0 += MF_BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < NA) *(bf16x8*)&As[srow[i]][scol[i]] = ra[i];
      *(bf16x8*)&Ws[srow[i]][scol[i]] = rw[i];
    }
    __syncthreads();
    const int kn = k0 + MF_BK;
    if (kn < K) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool ok = kn + scol[i] < K;
        if (i < NA) ra[i] = ok ? *(const bf16x8*)(ap[i] + kn) : zero;
        rw[i] = ok ? *(const bf16x8*)(wp[i] + kn) : zero;
      }
    }
#pragma unroll
    for (int kk = 0; kk < MF_BK / 16; ++kk) {
      const int kc = kk * 16 + lh * 8;
      const bf16x8 b0 = *(const bf16x8*)&Ws[wrow0][kc];
      const bf16x8 b1 = *(const bf16x8*)&Ws[wrow1][kc];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        const bf16x8 a = *(const bf16x8*)&As[arow + 32 * tm][kc];
        acc[tm][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, acc[tm][0], 0, 0, 0);
        acc[tm][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, acc[tm][1], 0, 0, 0);
      }
    }
    __syncthreads();
  }

  // lane holds C[row(v)][col]: row(v) = 8*(v/4) + 4*(lane/32) + v%4 inside a 32x32 tile, col = lane%32
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + wm * 32 * TM + tm * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
      if (m >= M) continue;
      if (EPI == MF_GATED) {
        const int n = n0 + wn * 32 + lr;
        if (n < N) {
          const float g = acc[tm][0][v];
          C[(long)m * ldc + n] = from_f32<TC>(g / (1.0f + __expf(-g)) * acc[tm][1][v]);
        }
      } else {
#pragma unroll
        for (int tn = 0; tn < 2; ++tn) {
          const int n = n0 + wn * 64 + tn * 32 + lr;
          if (n < N) {
            TC* c = C + (long)m * ldc + n;
            if (EPI == MF_ADD) *c = from_f32<TC>(to_f32<TC>(*c) + acc[tm][tn][v]);
            else *c = from_f32<TC>(acc[tm][tn][v]);
          }
        }
      }
    }
  }
}

template <int EPI, typename TC>
static int launch_mfma(const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw, long ldc,
                       hipStream_t stream) {
  const int ncols = (EPI == MF_GATED) ? 64 : 128;
  const int tiles_n = (N + ncols - 1) / ncols;
  // blocks of 128 rows unless that leaves fewer than two blocks per CU: then 64 rows, so that one
  // block's loads overlap another's products
  const bool tall = (long)((M + 127) / 128) * tiles_n >= 512;
  const int bm = tall ? 128 : 64;
  const int tiles_m = (M + bm - 1) / bm;
  const long n_tiles = (long)tiles_m * tiles_n;
  const long blocks = ((n_tiles + 7) / 8) * 8;
  GL3_REQUIRE(blocks < (1L << 31), "gl3_gemm_mfma: too many tiles");
  if (tall)
    gemm_mfma_kernel<EPI, TC, 2><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
        (const bf16_t*)A, (const bf16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, tiles_m, tiles_n);
  else
    gemm_mfma_kernel<EPI, TC, 1><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
        (const bf16_t*)A, (const bf16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, tiles_m, tiles_n);
  GL3_LAUNCH_CHECK();
  return 0;
}

// N counts output columns: for the gated epilogue W has 2N rows (gate, then up).
extern "C" int gl3_gemm_mfma(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, long lda, long ldw,
                             long ldc, int epilogue, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  GL3_REQUIRE(A && W && C && M > 0 && N > 0 && K > 0, "gl3_gemm_mfma: bad arguments (M=%d N=%d K=%d)", M, N, K);
  GL3_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gl3_gemm_mfma: K=%d, lda=%ld, ldw=%ld must be multiples of 8",
              K, lda, ldw);
  GL3_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "gl3_gemm_mfma: operands must be 16-byte aligned");
  GL3_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gl3_gemm_mfma: leading dimensions too small");
  GL3_REQUIRE(epilogue >= 0 && epilogue <= 2, "gl3_gemm_mfma: unknown epilogue %d", epilogue);
  GL3_REQUIRE(epilogue != MF_ADD || c_dtype == GL3_F32, "gl3_gemm_mfma: the add epilogue needs a float output");
  if (c_dtype == GL3_F32) {
    if (epilogue == MF_STORE) return launch_mfma<MF_STORE, float>(A, W, C, M, N, K, lda, ldw, ldc, stream);
    if (epilogue == MF_ADD) return launch_mfma<MF_ADD, float>(A, W, C, M, N, K, lda, ldw, ldc, stream);
    return launch_mfma<MF_GATED, float>(A, W, C, M, N, K, lda, ldw, ldc, stream);
  } else if (c_dtype == GL3_BF16) {
    if (epilogue == MF_STORE) return launch_mfma<MF_STORE, bf16_t>(A, W, C, M, N, K, lda, ldw, ldc, stream);
    if (epilogue == MF_GATED) return launch_mfma<MF_GATED, bf16_t>(A, W, C, M, N, K, lda, ldw, ldc, stream);
  }
  GL3_REQUIRE(false, "gl3_gemm_mfma: unsupported output dtype %d for epilogue %d", c_dtype, epilogue);
  return 0;
}

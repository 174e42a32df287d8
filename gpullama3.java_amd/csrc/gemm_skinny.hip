// C[M,N] = A[M,K] . W[N,K]^T in bfloat16 for few rows of A (M <= 64): the products of
// a decode step, where every weight is read once and the time is the time to stream W.
//
// Matrix cores, 16x16x32 tiles: the 16 rows of a strip of W are the tile's rows, up to
// 64 tokens (MT tiles of 16) its columns, so a lane's 16-byte load from W (8 consecutive
// k of one row) is the operand as the instruction wants it: W goes from memory to
// registers and nowhere else. A block is NW waves (4, 8 or 16) on one strip; wave w
// takes the k-steps w, w+NW, ... so that a strip's whole row range is in flight at
// once, and the NW partial tiles are summed through shared memory in wave order: the
// result has one fixed order of summation. K is never split across blocks: on this
// chip a block that waits for another block's stores has to push them through the
// per-XCD second-level caches, which costs more than the product itself.
//
// Epilogues as in gemm_generic.hip: store, add into a float matrix, gated
// (silu(gate) * up with the up rows `N` rows below the gate rows).
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

enum { SK_STORE = 0, SK_ADD = 1, SK_GATED = 2 };

#define SK_UNROLL 8

template <int MT, int NW, int EPI, typename TC>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                              TC* __restrict__ C, int M, int N, int K, long lda,
                                                              long ldw, long ldc) {
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  __shared__ f32x4 red[NW][NG * MT][64];
  const int strip = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int n0 = strip * 16;
  const int wr = min(n0 + r, N - 1);
  const bf16_t* wrow = W + (long)wr * ldw + q * 8;
  const bf16_t* urow = wrow + (long)N * ldw;  // up rows (gated only)
  const bf16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xrow[mt] = A + (long)min(mt * 16 + r, M - 1) * lda + q * 8;

  const int steps = (K + 31) / 32;   // k-steps of 32
  f32x4 acc[NG][MT];
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[g][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  for (int s0 = wave; s0 < steps; s0 += NW * SK_UNROLL) {
    bf16x8 wf[SK_UNROLL], uf[SK_UNROLL], xf[SK_UNROLL][MT];
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u) {
      const int k = (s0 + NW * u) * 32;
      const bool ok = k + q * 8 < K;   // K is a multiple of 8: a lane's 8 elements are all in or all out
      wf[u] = ok ? *(const bf16x8*)(wrow + k) : zero;
      if (EPI == SK_GATED) uf[u] = ok ? *(const bf16x8*)(urow + k) : zero;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xf[u][mt] = ok ? *(const bf16x8*)(xrow[mt] + k) : zero;
    }
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        acc[0][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u], xf[u][mt], acc[0][mt], 0, 0, 0);
        if (EPI == SK_GATED) acc[1][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[u], xf[u][mt], acc[1][mt], 0, 0, 0);
      }
    }
  }

  // the waves' partial tiles, summed in wave order by the wave that owns the tile
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
  // epilogue: lane holds C[mt*16 + r][n0 + 4q .. +3]
  for (int mt = wave; mt < MT; mt += NW) {
    const int m = mt * 16 + r;
    if (m >= M) continue;
    f32x4 v = red[0][mt][lane];
    if (EPI == SK_GATED) {
      const f32x4 up = red[0][MT + mt][lane];
#pragma unroll
      for (int c = 0; c < 4; ++c) v[c] = v[c] / (1.0f + __expf(-v[c])) * up[c];
    }
    const int n = n0 + 4 * q;
    TC* cp = C + (long)m * ldc + n;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (n + c < N) {
        if (EPI == SK_ADD) cp[c] = from_f32<TC>(to_f32<TC>(cp[c]) + v[c]);
        else cp[c] = from_f32<TC>(v[c]);
      }
    }
  }
}

template <int MT, int EPI, typename TC>
static int launch_skinny(int nw, const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw,
                         long ldc, hipStream_t stream) {
  constexpr int NG = (EPI == SK_GATED) ? 2 : 1;
  dim3 grid((N + 15) / 16);
#define GO(NW)                                                                                                       \
  gemm_skinny_kernel<MT, NW, EPI, TC><<<grid, dim3(NW * 64), 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (TC*)C, \
                                                                          M, N, K, lda, ldw, ldc)
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

template <int EPI, typename TC>
static int pick_mt(int mt, int nw, const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw,
                   long ldc, hipStream_t stream) {
  switch (mt) {
    case 1: return launch_skinny<1, EPI, TC>(nw, A, W, C, M, N, K, lda, ldw, ldc, stream);
    case 2: return launch_skinny<2, EPI, TC>(nw, A, W, C, M, N, K, lda, ldw, ldc, stream);
    case 3: return launch_skinny<3, EPI, TC>(nw, A, W, C, M, N, K, lda, ldw, ldc, stream);
    default: return launch_skinny<4, EPI, TC>(nw, A, W, C, M, N, K, lda, ldw, ldc, stream);
  }
}

// `waves`: waves per block wanted (4, 8, 16; 0 lets the library choose). Fewer are used when the
// partial tiles of that many waves would not fit the block's shared memory.
extern "C" int gl3_gemm_skinny(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, long lda,
                               long ldw, long ldc, int epilogue, int waves, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  GL3_REQUIRE(A && W && C, "gl3_gemm_skinny: null operand");
  GL3_REQUIRE(M > 0 && M <= 64, "gl3_gemm_skinny: M=%d is outside 1..64", M);
  GL3_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0,
              "gl3_gemm_skinny: K=%d, lda=%ld, ldw=%ld must be multiples of 8", K, lda, ldw);
  GL3_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "gl3_gemm_skinny: operands must be 16-byte aligned");
  GL3_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gl3_gemm_skinny: leading dimensions too small");
  GL3_REQUIRE(epilogue >= 0 && epilogue <= 2, "gl3_gemm_skinny: unknown epilogue %d", epilogue);
  GL3_REQUIRE(epilogue != SK_ADD || c_dtype == GL3_F32, "gl3_gemm_skinny: the add epilogue needs a float output");
  GL3_REQUIRE(waves == 0 || waves == 4 || waves == 8 || waves == 16, "gl3_gemm_skinny: waves=%d", waves);
  const int mt = (M + 15) / 16;
  if (waves == 0) {
    // enough waves to keep every CU's memory pipeline full, at least two k-steps each
    const long strips = (N + 15) / 16, steps = (K + 31) / 32;
    waves = 4;
    while (waves < 16 && strips * waves < 4096 && steps / (waves * 2) >= 2) waves *= 2;
  }
#define GO(EPI, TC) return pick_mt<EPI, TC>(mt, waves, A, W, C, M, N, K, lda, ldw, ldc, stream)
  if (c_dtype == GL3_F32) {
    if (epilogue == SK_STORE) GO(SK_STORE, float);
    if (epilogue == SK_ADD) GO(SK_ADD, float);
    GO(SK_GATED, float);
  } else if (c_dtype == GL3_BF16) {
    if (epilogue == SK_STORE) GO(SK_STORE, bf16_t);
    GO(SK_GATED, bf16_t);
  }
#undef GO
  GL3_REQUIRE(false, "gl3_gemm_skinny: unknown output dtype %d", c_dtype);
  return 0;
}

// C[M,N] = A[M,K] . W[N,K]^T for any sizes and any mix of float / bfloat16
// operands, with 32-bit multiply-adds only (no matrix-core, no reduced-precision
// mode): the true 32-bit path of the model and the fallback for shapes that the
// matrix-core kernels refuse. W is row-major [out, in] as the reference's matmul
// reads it (J/core/model/tensor/FloatTensor.java:98-100).
//
// Every output element is the sum over k = 0..K-1 in ascending order, one
// multiply-add per k, whatever M is and wherever the row sits in its tile: a
// token's result does not depend on how many tokens share the step.
//
// Epilogues: store (as float or bfloat16), add into a float matrix in place (the
// residual stream; the reference fuses the same, TransformerComputeKernelsLayered
// .java:766-784), and gated: W holds [gate rows | up rows] and the kernel writes
// act(gate) * up, act = silu as the reference's (J/inference/InferenceCore.java:158-166) or the tanh form
// of gelu. An optional bias per output column (float; gated: the gate's, then the up's) is added to
// the sums before anything else.
#include "common.h"

#define GT 64   // tile edge
#define GK 16   // k step

enum { EPI_STORE = 0, EPI_ADD = 1, EPI_GATED = 2 };

template <typename TA, typename TW, typename TC, int EPI>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                            TC* __restrict__ C, int M, int N, int K, long lda,
                                                            long ldw, long ldc, long up_offset,
                                                            const float* __restrict__ bias, int act, int w_order, int w_steps,
                                                            const int* __restrict__ w_pos) {
  // N is the number of output columns; for EPI_GATED the up rows of W start at
  // row `up_offset`. w_order, w_steps, w_pos: how W lies (gl3_w_offset).
  __shared__ float As[GK][GT + 1];
  __shared__ float Ws[GK][GT + 1];
  __shared__ float Us[EPI == EPI_GATED ? GK : 1][GT + 1];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;  // 16 x 16 threads, 4 x 4 outputs each
  const long m0 = (long)blockIdx.y * GT, n0 = (long)blockIdx.x * GT;
  float acc[4][4] = {};
  float accu[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GK) {
    // 64 x 16 elements per operand, 4 per thread; consecutive threads read along k
    for (int e = tid; e < GT * GK; e += 256) {
      const int r = e / GK, kk = e % GK;
      const int k = k0 + kk;
      float a = 0.f, w = 0.f, u = 0.f;
      if (k < K) {
        if (m0 + r < M) a = to_f32<TA>(A[(m0 + r) * lda + k]);
        if (n0 + r < N) {
          w = to_f32<TW>(W[gl3_w_offset(w_order, n0 + r, k, ldw, w_steps, w_pos)]);
          if (EPI == EPI_GATED) u = to_f32<TW>(W[gl3_w_offset(w_order, up_offset + n0 + r, k, ldw, w_steps, w_pos)]);
        }
      }
      As[kk][r] = a;
      Ws[kk][r] = w;
      if (EPI == EPI_GATED) Us[kk][r] = u;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float a[4], w[4], u[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
      if (EPI == EPI_GATED) {
#pragma unroll
        for (int j = 0; j < 4; ++j) u[j] = Us[kk][tx * 4 + j];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
          if (EPI == EPI_GATED) accu[i][j] = fmaf(a[i], u[j], accu[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias[n];
      if (EPI == EPI_GATED) {
        float u = accu[i][j];
        if (bias) u += bias[up_offset + n];
        v = gl3_activation<false>(v, act) * u;
      }
      TC* c = C + m * ldc + n;
      if (EPI == EPI_ADD) *c = from_f32<TC>(to_f32<TC>(*c) + v);
      else *c = from_f32<TC>(v);
    }
  }
}

template <typename TA, typename TW, typename TC>
static int launch_generic(const void* A, const void* W, void* C, int M, int N, int K, long lda, long ldw, long ldc,
                          int epi, const float* bias, int act, int w_order, int w_steps, const int* w_pos, hipStream_t stream) {
  dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT), block(256);
  GL3_REQUIRE(grid.y <= 65535, "gl3_gemm_generic: M=%d is too large for one launch", M);
  const TA* a = (const TA*)A;
  const TW* w = (const TW*)W;
  TC* c = (TC*)C;
  if (epi == EPI_STORE) gemm_generic_kernel<TA, TW, TC, EPI_STORE><<<grid, block, 0, stream>>>(a, w, c, M, N, K, lda, ldw, ldc, 0, bias, act, w_order, w_steps, w_pos);
  else if (epi == EPI_ADD) gemm_generic_kernel<TA, TW, TC, EPI_ADD><<<grid, block, 0, stream>>>(a, w, c, M, N, K, lda, ldw, ldc, 0, bias, act, w_order, w_steps, w_pos);
  else gemm_generic_kernel<TA, TW, TC, EPI_GATED><<<grid, block, 0, stream>>>(a, w, c, M, N, K, lda, ldw, ldc, N, bias, act, w_order, w_steps, w_pos);
  GL3_LAUNCH_CHECK();
  return 0;
}

// N counts output columns: for the gated epilogue W has 2N rows (gate, then up).
// bias (may be null): N floats (gated: 2N). act: the gated epilogue's activation (GL3_ACT_*).
// w_order, w_pos: how W lies (see below): as stored, or one of its copies in the matrix cores' order alone.
extern "C" int gl3_gemm_generic(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype, int M,
                                int N, int K, long lda, long ldw, long ldc, int epilogue, const float* bias, int act,
                                int w_order, const int* w_pos, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  GL3_REQUIRE(A && W && C && M > 0 && N > 0 && K > 0, "gl3_gemm_generic: bad arguments (M=%d N=%d K=%d)", M, N, K);
  GL3_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gl3_gemm_generic: leading dimensions %ld %ld %ld too small", lda, ldw, ldc);
  GL3_REQUIRE(epilogue >= 0 && epilogue <= 2, "gl3_gemm_generic: unknown epilogue %d", epilogue);
  GL3_REQUIRE(epilogue != EPI_ADD || c_dtype == GL3_F32, "gl3_gemm_generic: the add epilogue needs a float output");
  GL3_REQUIRE(act == GL3_ACT_SILU || act == GL3_ACT_GELU_TANH, "gl3_gemm_generic: unknown activation %d", act);
  // w_order: 0: W holds the rows as stored. 1: W is the copy in the matrix operands' order (lib.tile_weight); w_pos (may be
  // null) then names each row's place in it. 2: the copy in packed strips of 8 rows (lib.tile_weight8).
  const long w_rows = epilogue == EPI_GATED ? 2L * N : N;
  GL3_REQUIRE(w_order >= 0 && w_order <= 2 && (w_order != 1 || w_rows % 16 == 0) && (w_order != 2 || w_rows % 8 == 0) &&
                  (w_order == 1 || !w_pos),
              "gl3_gemm_generic: W in order %d with N=%d, epilogue %d", w_order, N, epilogue);
  const int w_steps = w_order == 1 ? (K + 31) / 32 : (K + 63) / 64;
  const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
  switch (key) {
    case 0: return launch_generic<float, float, float>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, bias, act, w_order, w_steps, w_pos, stream);
    case 2: return launch_generic<float, bf16_t, float>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, bias, act, w_order, w_steps, w_pos, stream);
    case 4: return launch_generic<bf16_t, float, float>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, bias, act, w_order, w_steps, w_pos, stream);
    case 5: return launch_generic<bf16_t, float, bf16_t>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, bias, act, w_order, w_steps, w_pos, stream);
    case 6: return launch_generic<bf16_t, bf16_t, float>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, bias, act, w_order, w_steps, w_pos, stream);
    case 7: return launch_generic<bf16_t, bf16_t, bf16_t>(A, W, C, M, N, K, lda, ldw, ldc, epilogue, bias, act, w_order, w_steps, w_pos, stream);
    default:
      GL3_REQUIRE(false, "gl3_gemm_generic: unsupported dtypes A=%d W=%d C=%d", a_dtype, w_dtype, c_dtype);
  }
  return 0;
}

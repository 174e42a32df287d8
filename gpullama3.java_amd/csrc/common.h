// Shared device helpers for the gfx950 kernels: element types, conversions,
// wave64 reductions, and the error convention of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

#define GL3_WAVE 64

// ---- error convention: every entry point returns 0 or a negative code and
// leaves a message that gl3_last_error() returns.
extern "C" const char* gl3_last_error();
void gl3_set_error(const char* fmt, ...);

#define GL3_REQUIRE(cond, ...)            \
  do {                                    \
    if (!(cond)) {                        \
      gl3_set_error(__VA_ARGS__);         \
      return -1;                          \
    }                                     \
  } while (0)

#define GL3_LAUNCH_CHECK()                                              \
  do {                                                                  \
    hipError_t e__ = hipGetLastError();                                 \
    if (e__ != hipSuccess) {                                            \
      gl3_set_error("%s: launch failed: %s", __func__, hipGetErrorString(e__)); \
      return -2;                                                        \
    }                                                                   \
  } while (0)

// dtype codes shared with the Python side
enum { GL3_F32 = 0, GL3_BF16 = 1 };

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return static_cast<float>(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return static_cast<bf16_t>(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of shared memory. The order of the sum
// depends only on the block size.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += scratch[i];
  return t;
}
__device__ __forceinline__ double block_sum_f64(double v, double* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = wave_sum_f64(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  double t = 0.0;
  for (int i = 0; i < nw; ++i) t += scratch[i];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
  for (int i = 1; i < nw; ++i) t = fmaxf(t, scratch[i]);
  return t;
}

// ---- what a product's epilogue may apply besides its own rule: a bias per output column (float;
// for the gated epilogue the gate's biases, then the up's), and the activation of the gated
// epilogue. The reference's feed-forward is silu without biases (J/inference/InferenceCore.java:158-166).
// How one kv head's keys and values lie inside a page of the cache. A key page holds
// [position][head_dim] elements, a value page [head_dim][position] (transposed), but not row by
// row: in tiles of 16 rows x 8 columns (16 bytes of bfloat16 a row), the tiles of the same 16 rows
// one after another along the columns. A matrix-core operand (lane r, q: row r, the 8 elements at
// column block q) of 16 rows x 32 columns is then 1 KB of consecutive memory in lane order, where
// rows lying one after another would make every lane touch a line of its own, which costs a CU's
// first-level cache four times the time.
//   values: tile (dim / 16, position / 8), row dim % 16, element position % 8
//   keys:   32 positions make two tiles: the positions with bit 2 clear, then those with it set, so
//           row i of the first is position 8 * (i / 4) + i % 4 of the 32 and row i of the second the
//           position 4 further. (The decode kernel's two score tiles of a chunk of 32 keys: a lane
//           then holds the probabilities of 8 consecutive keys, one 16-byte load of a value row.)
// page_size is a multiple of 32, head_dim of 16; 32 positions of a key page are still 32 * head_dim
// consecutive elements, and 8 elements that are consecutive along a row stay consecutive.
__device__ __forceinline__ long gl3_k_offset(int position_in_page, int dim, int head_dim) {
  const int p = position_in_page;
  const int tile = (p >> 5) * 2 + ((p >> 2) & 1), row = ((p >> 3) & 3) * 4 + (p & 3);
  return ((long)(tile * (head_dim >> 3) + (dim >> 3)) << 7) + (row << 3) + (dim & 7);
}
__device__ __forceinline__ long gl3_v_offset(int dim, int position_in_page, int page_size) {
  return ((long)((dim >> 4) * (page_size >> 3) + (position_in_page >> 3)) << 7) + ((dim & 15) << 3) + (position_in_page & 7);
}

// Element (row n, column k) of a matrix that is kept in the order of the matrix operands:
// [strip of 16 rows][k-step of 32][lane = 16 * (k block of 8) + row][8 elements], `steps` k-steps a strip
// (lib.tile_weight; 8 consecutive k of a row lie together).
__host__ __device__ __forceinline__ long gl3_operand_offset(long n, int k, int steps) {
  return (((n >> 4) * steps + (k >> 5)) << 9) + (((k & 31) >> 3) << 7) + ((n & 15) << 3) + (k & 7);
}
// The same for the packed strips of 8 rows: [strip of 8 rows][step of 64 k][lane = 16 * (k block of 8 inside its
// half) + 8 * (half of the step) + row][8 elements], `steps` steps of 64 a strip (lib.tile_weight8).
__host__ __device__ __forceinline__ long gl3_packed_offset(long n, int k, int steps) {
  return (((n >> 3) * steps + (k >> 6)) << 9) + (((k & 31) >> 3) << 7) + (((k >> 5) & 1) << 6) + ((n & 7) << 3) + (k & 7);
}
// Where element (n, k) of W lies. order 0: rows as stored (ldw); 1: the operands' order; 2: the packed strips of 8.
// `pos` (order 1, may be null): the place of each row in a copy whose strips hold the rows in another order.
__host__ __device__ __forceinline__ long gl3_w_offset(int order, long n, int k, long ldw, int steps, const int* pos) {
  if (order == 0) return n * ldw + k;
  if (order == 1) return gl3_operand_offset(pos ? pos[n] : n, k, steps);
  return gl3_packed_offset(n, k, steps);
}

enum { GL3_ACT_SILU = 0, GL3_ACT_GELU_TANH = 1 };

template <bool FAST>
__device__ __forceinline__ float gl3_activation(float v, int act) {
  if (act == GL3_ACT_GELU_TANH) {
    // 0.5 v (1 + tanh(sqrt(2/pi) (v + 0.044715 v^3))) = v / (1 + exp(-2 u))
    const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
    return v / (1.0f + (FAST ? __expf(-2.0f * u) : expf(-2.0f * u)));
  }
  return v / (1.0f + (FAST ? __expf(-v) : expf(-v)));
}

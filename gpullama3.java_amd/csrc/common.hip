#include "common.h"
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

void gl3_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* gl3_last_error() { return g_error; }

extern "C" int gl3_abi_version() { return 1; }

// ---- fill: clears or sets a buffer with a kernel (a memset node is not safe
// inside a captured graph on this platform).
__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, long n) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

extern "C" int gl3_fill_u32(void* p, uint32_t v, long n, hipStream_t stream) {
  if (n <= 0) return 0;
  GL3_REQUIRE(p != nullptr, "gl3_fill_u32: null pointer");
  long blocks = (n + 255) / 256;
  GL3_REQUIRE(blocks < (1L << 31), "gl3_fill_u32: %ld words is too many", n);
  fill_u32_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>((uint32_t*)p, v, n);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ---- p[i] *= s (what a model's logit scale is applied with)
__global__ void scale_f32_kernel(float* p, float s, long n) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] *= s;
}

extern "C" int gl3_scale_f32(float* p, float s, long n, hipStream_t stream) {
  if (n <= 0) return 0;
  GL3_REQUIRE(p != nullptr, "gl3_scale_f32: null pointer");
  long blocks = (n + 255) / 256;
  GL3_REQUIRE(blocks < (1L << 31), "gl3_scale_f32: %ld elements is too many", n);
  scale_f32_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(p, s, n);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ---- p[i] = cap * tanh(p[i] / cap) (what a model's soft cap of the logits is applied with)
__global__ void softcap_f32_kernel(float* p, float cap, long n) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = cap * tanhf(p[i] / cap);
}

extern "C" int gl3_softcap_f32(float* p, float cap, long n, hipStream_t stream) {
  if (n <= 0) return 0;
  GL3_REQUIRE(p != nullptr && cap > 0.f, "gl3_softcap_f32: null pointer or a cap that is not positive");
  long blocks = (n + 255) / 256;
  GL3_REQUIRE(blocks < (1L << 31), "gl3_softcap_f32: %ld elements is too many", n);
  softcap_f32_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(p, cap, n);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ---- scatter of a few integers whose places and values travel in the launch itself: how the host
// changes entries of a table on the device (a page added to a sequence) without staging memory.
#define GL3_SCATTER_MAX 128
struct ScatterArgs { int idx[GL3_SCATTER_MAX]; int val[GL3_SCATTER_MAX]; };

__global__ void scatter_i32_kernel(int* dst, int n, ScatterArgs a) {
  const int i = threadIdx.x;
  if (i < n) dst[a.idx[i]] = a.val[i];
}

// dst[idx[i]] = val[i] for i < n (host arrays); `limit`: elements of dst, every idx is checked against it.
extern "C" int gl3_scatter_i32(int* dst, long limit, const int* idx, const int* val, int n, hipStream_t stream) {
  if (n <= 0) return 0;
  GL3_REQUIRE(dst && idx && val, "gl3_scatter_i32: null argument");
  for (int i = 0; i < n; ++i)
    GL3_REQUIRE(idx[i] >= 0 && idx[i] < limit, "gl3_scatter_i32: place %d is outside the %ld elements", idx[i], limit);
  for (int lo = 0; lo < n; lo += GL3_SCATTER_MAX) {
    ScatterArgs a;
    const int m = n - lo < GL3_SCATTER_MAX ? n - lo : GL3_SCATTER_MAX;
    for (int i = 0; i < m; ++i) { a.idx[i] = idx[lo + i]; a.val[i] = val[lo + i]; }
    for (int i = m; i < GL3_SCATTER_MAX; ++i) { a.idx[i] = 0; a.val[i] = 0; }
    scatter_i32_kernel<<<dim3(1), dim3(GL3_SCATTER_MAX), 0, stream>>>(dst, m, a);
    GL3_LAUNCH_CHECK();
  }
  return 0;
}

// ---- a copy from pinned host memory to the device on a stream (one call, no tensor objects)
extern "C" int gl3_upload(void* dst, const void* src, long bytes, hipStream_t stream) {
  if (bytes <= 0) return 0;
  GL3_REQUIRE(dst && src, "gl3_upload: null argument");
  hipError_t e = hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyHostToDevice, stream);
  GL3_REQUIRE(e == hipSuccess, "gl3_upload: %s", hipGetErrorString(e));
  return 0;
}

// ---- the input of a decode step, written into the device buffer that a captured step reads. The
// numbers travel in the launch itself (no staging memory, nothing to wait for before the host may
// write the next step's): tokens | positions | tokens held before (the same numbers) | slots, each
// `n_pad` long; entries from `n` on are padding: token 0 at position 0 of slot `pad_slot`.
#define GL3_STAGE_MAX 256
struct StageArgs { int tok[GL3_STAGE_MAX]; int pos[GL3_STAGE_MAX]; int slot[GL3_STAGE_MAX]; };

__global__ void stage_decode_kernel(int* dst, int n_pad, int first, int count, int n, int pad_slot, int* counter,
                                    StageArgs a) {
  const int i = threadIdx.x;
  if (i < count) {
    const int e = first + i;
    const bool real = e < n;
    dst[e] = real ? a.tok[i] : 0;
    dst[n_pad + e] = real ? a.pos[i] : 0;
    dst[2 * n_pad + e] = real ? a.pos[i] : 0;
    dst[3 * n_pad + e] = real ? a.slot[i] : pad_slot;
  }
  if (i == 0 && first == 0 && counter) counter[0] = 0;
}

// tokens, positions, slots: host arrays of n entries. dst: device, at least 4 * n_pad ints. counter (may be
// null): a device int set to 0 (the step counter of a run of steps).
extern "C" int gl3_stage_decode(int* dst, int n_pad, int n, const int* tokens, const int* positions, const int* slots,
                                int pad_slot, int* counter, hipStream_t stream) {
  GL3_REQUIRE(dst && tokens && positions && slots && n >= 0 && n <= n_pad && n_pad > 0, "gl3_stage_decode: bad arguments");
  for (int first = 0; first < n_pad; first += GL3_STAGE_MAX) {
    StageArgs a;
    const int count = n_pad - first < GL3_STAGE_MAX ? n_pad - first : GL3_STAGE_MAX;
    for (int i = 0; i < count; ++i) {
      const int e = first + i;
      a.tok[i] = e < n ? tokens[e] : 0;
      a.pos[i] = e < n ? positions[e] : 0;
      a.slot[i] = e < n ? slots[e] : pad_slot;
    }
    stage_decode_kernel<<<dim3(1), dim3(GL3_STAGE_MAX), 0, stream>>>(dst, n_pad, first, count, n, pad_slot, counter, a);
    GL3_LAUNCH_CHECK();
  }
  return 0;
}

// ---- the input of a step that brings any number of tokens per sequence. The host names, per entry, its
// slot, the tokens its sequence holds already and the tokens it brings; what the kernels read per TOKEN
// (position, sequence, row of the block table) is expanded on the device. The host's part travels as one
// copy from pinned memory, laid out as the device buffer's head:
//   tokens[T] | cu_seqlens[B+1] | kv_before[B] | slots[B] | wanted rows[W] | positions[T] | seq_of_token[T] | table_rows[T]
// (the last three are written by the kernel). The caller owns `pinned` until the copy has run.
__global__ void expand_step_kernel(const int* __restrict__ cu, const int* __restrict__ kv_before,
                                   const int* __restrict__ slots, int B, int T, int* __restrict__ positions,
                                   int* __restrict__ seq_of, int* __restrict__ table_rows) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  int lo = 0, hi = B - 1;                 // the entry b with cu[b] <= t < cu[b + 1]
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid - 1;
  }
  positions[t] = kv_before[lo] + (t - cu[lo]);
  seq_of[t] = lo;
  table_rows[t] = slots[lo];
}

extern "C" long gl3_stage_step_ints(int T, int B, int W) { return 4L * T + 3L * B + 1 + W; }

// tokens: T host ints (the entries' tokens one after another); slots, starts, counts: B host ints; want: W packed
// rows. vocab: every token is checked against it. dev: device, gl3_stage_step_ints(T, B, W) ints; pinned: host
// memory that the device can read, T + 3 B + 1 + W ints.
extern "C" int gl3_stage_step(int* dev, int* pinned, const int* tokens, int T, const int* slots, const int* starts,
                              const int* counts, int B, const int* want, int W, int vocab, hipStream_t stream) {
  GL3_REQUIRE(dev && pinned && tokens && slots && starts && counts && T > 0 && B > 0 && W >= 0 && (want || W == 0),
              "gl3_stage_step: bad arguments");
  int* cu = pinned + T;
  int* before = cu + B + 1;
  int* sl = before + B;
  int* wr = sl + B;
  cu[0] = 0;
  for (int b = 0; b < B; ++b) {
    GL3_REQUIRE(counts[b] > 0 && starts[b] >= 0, "gl3_stage_step: entry %d brings %d tokens at %d", b, counts[b], starts[b]);
    cu[b + 1] = cu[b] + counts[b];
    before[b] = starts[b];
    sl[b] = slots[b];
  }
  GL3_REQUIRE(cu[B] == T, "gl3_stage_step: the entries bring %d tokens, %d were given", cu[B], T);
  for (int t = 0; t < T; ++t) {
    const int v = tokens[t];
    GL3_REQUIRE(v >= 0 && v < vocab, "gl3_stage_step: token id %d is outside the vocabulary of %d", v, vocab);
    pinned[t] = v;
  }
  for (int i = 0; i < W; ++i) {
    GL3_REQUIRE(want[i] >= 0 && want[i] < T, "gl3_stage_step: wanted row %d of %d", want[i], T);
    wr[i] = want[i];
  }
  const long head = (long)T + 3L * B + 1 + W;
  hipError_t e = hipMemcpyAsync(dev, pinned, (size_t)head * sizeof(int), hipMemcpyHostToDevice, stream);
  GL3_REQUIRE(e == hipSuccess, "gl3_stage_step: %s", hipGetErrorString(e));
  int* d_cu = dev + T;
  int* d_pos = dev + head;
  expand_step_kernel<<<dim3((T + 255) / 256), dim3(256), 0, stream>>>(d_cu, d_cu + B + 1, d_cu + 2 * B + 1, B, T, d_pos,
                                                                      d_pos + T, d_pos + 2 * T);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ---- launch of an instantiated graph (a captured decode step) on a stream
extern "C" int gl3_graph_launch(void* graph_exec, hipStream_t stream) {
  GL3_REQUIRE(graph_exec, "gl3_graph_launch: null graph");
  hipError_t e = hipGraphLaunch((hipGraphExec_t)graph_exec, stream);
  GL3_REQUIRE(e == hipSuccess, "gl3_graph_launch: %s", hipGetErrorString(e));
  return 0;
}

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

// ---- touch: reads a range of memory and keeps nothing, so that the range lies in the
// memory-side cache when the kernel that needs it starts. `blocks` blocks of 256 threads walk
// over the range in 16-byte loads, eight in flight per thread. The sink is written only if every
// word read is one bit pattern that no weight holds: it keeps the loads alive.
__global__ __launch_bounds__(256) void touch_kernel(const uint4* __restrict__ p, long n16, uint32_t* __restrict__ sink) {
  const long stride = (long)gridDim.x * blockDim.x;
  uint32_t seen = 0xffffffffu;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += 8 * stride) {
    uint4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = i + u * stride < n16 ? p[i + u * stride] : uint4{0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < 8; ++u) seen &= v[u].x & v[u].y & v[u].z & v[u].w;
  }
  if (seen == 0xffffffffu && n16 > (1L << 60)) *sink = seen;
}

extern "C" int gl3_touch(const void* p, long bytes, int blocks, void* sink, hipStream_t stream) {
  if (bytes <= 0) return 0;
  GL3_REQUIRE(p && sink && (uintptr_t)p % 16 == 0, "gl3_touch: null or unaligned pointer");
  GL3_REQUIRE(blocks > 0 && blocks <= 65536, "gl3_touch: %d blocks", blocks);
  touch_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>((const uint4*)p, bytes / 16, (uint32_t*)sink);
  GL3_LAUNCH_CHECK();
  return 0;
}

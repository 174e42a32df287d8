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

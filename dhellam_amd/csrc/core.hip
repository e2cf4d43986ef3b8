// Library-wide pieces: version, per-thread error message, calibration copy kernel.
#include "common.h"
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

namespace dh {
static thread_local char g_err[1024] = "";

void set_error(const char *file, int line, const char *func, const char *fmt, ...) {
  const char *base = strrchr(file, '/');
  base = base ? base + 1 : file;
  int n = snprintf(g_err, sizeof(g_err), "%s:%d in function %s: ", base, line, func);
  if (n < 0) n = 0;
  if (n >= (int)sizeof(g_err)) return;
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err + n, sizeof(g_err) - n, fmt, ap);
  va_end(ap);
}
}  // namespace dh

extern "C" int dh_version(void) { return 100; }
extern "C" const char *dh_last_error(void) { return dh::g_err; }

// Grid-stride 16-byte copy; the tail (nbytes % 16) is copied bytewise by block 0.
__global__ void __launch_bounds__(256) copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                   int64_t nvec, const uint8_t *src_tail, uint8_t *dst_tail,
                                                   int ntail) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < nvec; i += stride) dst[i] = src[i];
  if (blockIdx.x == 0 && (int)threadIdx.x < ntail) dst_tail[threadIdx.x] = src_tail[threadIdx.x];
}

extern "C" int dh_copy_bytes(const void *src, void *dst, int64_t nbytes, void *stream) {
  DH_CHECK(nbytes >= 0, "nbytes must be >= 0");
  if (nbytes == 0) return DH_OK;
  DH_CHECK(src && dst, "null pointer");
  DH_CHECK(dh::aligned16(src) && dh::aligned16(dst), "src/dst must be 16-byte aligned");
  const int64_t nvec = nbytes / 16;
  const int ntail = (int)(nbytes % 16);
  int64_t blocks = dh::cdiv(nvec, 256 * 4);
  if (blocks < 1) blocks = 1;
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const uint4 *)src, (uint4 *)dst, nvec, (const uint8_t *)src + nvec * 16,
                     (uint8_t *)dst + nvec * 16, ntail);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

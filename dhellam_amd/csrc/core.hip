// Library-wide pieces: version, per-thread error message, calibration copy kernel.
#include "common.h"
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#include <algorithm>
#include <mutex>
#include <vector>

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

extern "C" int dh_version(void) { return 200; }
extern "C" const char *dh_last_error(void) { return dh::g_err; }

// Grid-stride 16-byte copy; the tail (nbytes % 16) is copied bytewise by block 0.
template <bool NT>
__global__ void __launch_bounds__(256) copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                   int64_t nvec, const uint8_t *src_tail, uint8_t *dst_tail,
                                                   int ntail) {
  // Each trip a workgroup moves one contiguous 16 KB run: four 16-byte vectors per lane, 4 KB apart.
  using V = dh::Vec<uint32_t>;
  const uint32_t *s = reinterpret_cast<const uint32_t *>(src);
  uint32_t *d = reinterpret_cast<uint32_t *>(dst);
  const int64_t step = (int64_t)gridDim.x * 1024;
  for (int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x; i < nvec; i += step) {
    V v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + u * 256 < nvec) v[u] = dh::ldg_s<NT>(s + (i + u * 256) * 4);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + u * 256 < nvec) dh::stg_s<NT>(d + (i + u * 256) * 4, v[u]);
  }
  if (blockIdx.x == 0 && (int)threadIdx.x < ntail) dst_tail[threadIdx.x] = src_tail[threadIdx.x];
}

// One wavefront that does nothing for `ticks` ticks of the constant 100 MHz clock.  Bounded twice: by the
// clock and by an iteration count, so it always ends.
__global__ void __launch_bounds__(64) delay_kernel(unsigned long long ticks, unsigned long long max_iters) {
  const unsigned long long t0 = wall_clock64();
  for (unsigned long long i = 0; i < max_iters; ++i) {
    if (wall_clock64() - t0 >= ticks) break;
    __builtin_amdgcn_s_sleep(32);
  }
}

extern "C" int dh_delay(int64_t nanoseconds, void *stream) {
  DH_CHECK(nanoseconds >= 0 && nanoseconds <= 1000000000ll, "delay of %lld ns outside [0, 1 s]", (long long)nanoseconds);
  if (nanoseconds == 0) return DH_OK;
  const unsigned long long ticks = (unsigned long long)(nanoseconds / 10);             // 100 MHz
  // one iteration sleeps 32 x 64 cycles, at least 0.8 us at any engine clock: 4 x the iterations that fill the time
  const unsigned long long max_iters = (unsigned long long)(nanoseconds / 200) + 1024;
  hipLaunchKernelGGL(delay_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, ticks, max_iters);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

// The same stretch of stream time without a compute unit: a host function in the stream, which the runtime calls on
// one of its own threads once the stream's earlier work is done and whose return releases the work behind it.  It
// stands for a transfer that an agent other than the compute units carries (a copy engine, a network adapter):
// unlike the delay kernel it needs no free wavefront slot, so it starts while a kernel of another stream owns every
// compute unit.  What it costs the stream beyond the requested time is the runtime's hand-over to its thread and
// back (measured by the caller, not assumed).
namespace dh {
static void host_spin_entry(void *arg) {
  const int64_t ns = (int64_t)(intptr_t)arg;
  timespec t0, t;
  clock_gettime(CLOCK_MONOTONIC, &t0);
  for (;;) {
    clock_gettime(CLOCK_MONOTONIC, &t);
    if ((int64_t)(t.tv_sec - t0.tv_sec) * 1000000000ll + (t.tv_nsec - t0.tv_nsec) >= ns) break;
  }
}
}  // namespace dh

extern "C" int dh_host_delay(int64_t nanoseconds, void *stream) {
  DH_CHECK(nanoseconds >= 0 && nanoseconds <= 1000000000ll, "delay of %lld ns outside [0, 1 s]", (long long)nanoseconds);
  if (nanoseconds == 0) return DH_OK;
  DH_HIP(hipLaunchHostFunc((hipStream_t)stream, dh::host_spin_entry, (void *)(intptr_t)nanoseconds));
  return DH_OK;
}

// Masked streams that are alive, and their owner of last resort.  A caller that wraps such a stream in an object
// that only borrows the handle (torch's ExternalStream) and never calls dh_stream_destroy would leave it open
// until the HIP runtime's own exit-time destructors run; with a profiler attached (rocprofv3), whose tool has
// finalised by then, a process that had made four of them ended with SIGSEGV after printing its result.
// The first creation therefore registers an exit handler.  Handlers run in reverse order of registration, so
// this one runs before those of the runtime and of a preloaded tool (both registered at load time) and after
// the host program's own shutdown (a Python interpreter has freed its tensors by then: a tensor freed AFTER a
// stream it was used on is destroyed would make the caching allocator record an event on a dead stream).
namespace dh {
static std::mutex g_streams_mutex;
static std::vector<hipStream_t> g_masked_streams;
static bool g_exit_hook = false;

static void destroy_masked_streams_at_exit() {
  std::vector<hipStream_t> left;
  {
    std::lock_guard<std::mutex> lock(g_streams_mutex);
    left.swap(g_masked_streams);
  }
  for (hipStream_t st : left) {
    if (hipStreamSynchronize(st) == hipSuccess) (void)hipStreamDestroy(st);
  }
}
}  // namespace dh

// A stream whose kernels run only on the compute units whose bit is set in `mask` (bit i of word i / 32;
// on a device with several XCDs bit i is compute unit i / n_xcd of XCD i % n_xcd).
extern "C" int dh_stream_create_cu_mask(const uint32_t *mask, int words, void **stream_out) {
  DH_CHECK(mask && stream_out, "null pointer");
  int dev = 0, cus = 0;
  DH_HIP(hipGetDevice(&dev));
  DH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  DH_CHECK(words >= 1 && words * 32 >= cus && words <= 64, "mask of %d words does not cover the device's %d compute units", words, cus);
  int set = 0;
  for (int i = 0; i < cus; ++i) set += (mask[i / 32] >> (i % 32)) & 1;
  DH_CHECK(set > 0, "the mask enables no compute unit");
  hipStream_t st = nullptr;
  DH_HIP(hipExtStreamCreateWithCUMask(&st, (uint32_t)words, mask));
  {
    std::lock_guard<std::mutex> lock(dh::g_streams_mutex);
    dh::g_masked_streams.push_back(st);
    if (!dh::g_exit_hook) {
      dh::g_exit_hook = true;
      atexit(dh::destroy_masked_streams_at_exit);
    }
  }
  *stream_out = (void *)st;
  return DH_OK;
}

extern "C" int dh_stream_destroy(void *stream) {
  DH_CHECK(stream, "null stream");
  {
    std::lock_guard<std::mutex> lock(dh::g_streams_mutex);
    auto &v = dh::g_masked_streams;
    auto it = std::find(v.begin(), v.end(), (hipStream_t)stream);
    DH_CHECK(it != v.end(), "not a live stream of dh_stream_create_cu_mask (destroyed twice?)");
    v.erase(it);
  }
  DH_HIP(hipStreamDestroy((hipStream_t)stream));
  return DH_OK;
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
  if (blocks > 65536) blocks = 65536;
  if (dh::stream_hint(2 * nbytes))
    hipLaunchKernelGGL(copy_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const uint4 *)src, (uint4 *)dst, nvec, (const uint8_t *)src + nvec * 16,
                       (uint8_t *)dst + nvec * 16, ntail);
  else
    hipLaunchKernelGGL(copy_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const uint4 *)src, (uint4 *)dst, nvec, (const uint8_t *)src + nvec * 16,
                       (uint8_t *)dst + nvec * 16, ntail);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

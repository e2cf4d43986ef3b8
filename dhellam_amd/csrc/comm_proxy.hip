// A resident communication proxy: the stand-in for collectives that a stream can post and wait for WITHOUT
// launching a kernel per collective.
//
// Why: a kernel launched while a large GEMM of another stream owns every compute unit is placed only after that
// GEMM has placed its last workgroup, so a 55 us collective posted as a kernel of its own next to such a GEMM
// takes 150-400 us, and the double-strand schedule hides none of it.  The proxy is ONE kernel, launched at the
// start of a step: one wavefront per slot (a slot = a strand's communication channel) that sleeps until a
// request arrives, carries it out, and reports it done.  A strand posts a request with a stream write
// (hipStreamWriteValue32) and blocks behind it with a stream wait (hipStreamWaitValue32): both are carried out by
// the command processor, no compute unit and no kernel dispatch is involved, so the request is seen within
// microseconds whatever else is running, and the other strand's kernels keep the chip busy meanwhile.  It plays
// the role the reference gives its third stream and communication handles (dhellam/core/dstb.py:1142-1188: the
// collective is posted on stream 3, the compute op waits for its handle).
//
// On one GPU there is nothing to transfer: a request is carried out by waiting for the duration the collective
// would take (as dh_delay does).  Every wait of the kernel is bounded: a slot gives up after `limit_ns` without a
// request or a stop, and when it gives up it publishes a "done" count that releases every stream wait behind it.
#include <mutex>
#include <vector>

#include "common.h"

namespace dh {

constexpr int PROXY_MAX_SLOTS = 8;
constexpr int PROXY_LOG = 256;   // per slot: (start, end) clock stamps of the first collectives of the last launch

// The flags, one 8-byte piece of signal memory each (the kind of memory the command processor can wait on; it is
// handed out in pieces of exactly that size).  They stay allocated until the process ends.
struct ProxyFlags {
  uint32_t *req[PROXY_MAX_SLOTS];    // requests posted so far        (stream write -> kernel)
  uint32_t *done[PROXY_MAX_SLOTS];   // requests carried out so far   (kernel -> stream wait)
  uint32_t *stop[PROXY_MAX_SLOTS];   // number of the launch that may end once it has nothing pending
};

struct CommProxy {
  int slots = 0;
  int device = 0;
  ProxyFlags f{};
  unsigned long long *log = nullptr;          // device, [slots][PROXY_LOG][2]
  uint32_t posted[PROXY_MAX_SLOTS] = {};      // host mirror of req
  uint32_t launch_no = 0;                     // launches so far
  bool running = false;                       // a launch has not been told to stop yet
};

// slot = blockIdx.x; lane 0 works, the rest of the wavefront leaves at once.
__global__ void __launch_bounds__(64)
comm_proxy_kernel(ProxyFlags f, unsigned long long *log, uint32_t launch_no, unsigned long long dur_ticks,
                  unsigned long long limit_ticks) {
  if (threadIdx.x != 0) return;
  const int s = blockIdx.x;
  uint32_t served = __hip_atomic_load(f.done[s], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const uint32_t first = served;
  unsigned long long idle_since = wall_clock64();
  for (;;) {
    const uint32_t r = __hip_atomic_load(f.req[s], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    if ((int32_t)(r - served) > 0) {                     // a request: carry it out
      const unsigned long long t0 = wall_clock64();
      // bounded twice: by the clock and by an iteration count (an iteration sleeps 8 x 64 cycles, >= 0.2 us)
      const unsigned long long max_iters = dur_ticks / 8 + 1024;
      for (unsigned long long i = 0; i < max_iters; ++i) {
        if (wall_clock64() - t0 >= dur_ticks) break;
        __builtin_amdgcn_s_sleep(8);
      }
      ++served;
      const uint32_t k = served - first - 1;
      if (k < (uint32_t)PROXY_LOG) {
        log[((size_t)s * PROXY_LOG + k) * 2] = t0;
        log[((size_t)s * PROXY_LOG + k) * 2 + 1] = wall_clock64();
      }
      __hip_atomic_store(f.done[s], served, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
      idle_since = wall_clock64();
      continue;
    }
    // Nothing pending.  Leave if this launch was told to stop: the stop is written in stream order behind the
    // strand's last request, so no request of this launch can arrive after it.  Leave, too, if nothing at all came
    // for too long, and then report every request that could still come as done, so that no stream stays blocked
    // behind a proxy that is gone (such a collective then took no time: wrong, but it ends).
    const uint32_t st = __hip_atomic_load(f.stop[s], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    if (st == launch_no) break;
    if (wall_clock64() - idle_since >= limit_ticks) {
      __hip_atomic_store(f.done[s], served + 0x40000000u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
      break;
    }
    __builtin_amdgcn_s_sleep(4);
  }
}

static int proxy_check(const CommProxy *p, int slot) {
  DH_CHECK(p != nullptr, "null proxy");
  DH_CHECK(slot >= 0 && slot < p->slots, "slot %d outside [0, %d)", slot, p->slots);
  return DH_OK;
}

static int flag_alloc(uint32_t **out) {
  void *p = nullptr;
  DH_HIP(hipExtMallocWithFlags(&p, 8, hipMallocSignalMemory));
  DH_HIP(hipMemset(p, 0, 8));
  *out = (uint32_t *)p;
  return DH_OK;
}

}  // namespace dh

extern "C" int dh_comm_proxy_create(int slots, void **proxy_out) {
  using namespace dh;
  DH_CHECK(proxy_out != nullptr, "null pointer");
  DH_CHECK(slots >= 1 && slots <= PROXY_MAX_SLOTS, "slots=%d outside [1, %d]", slots, PROXY_MAX_SLOTS);
  CommProxy *p = new CommProxy();
  p->slots = slots;
  DH_HIP(hipGetDevice(&p->device));
  for (int s = 0; s < PROXY_MAX_SLOTS; ++s) {      // unused slots point at slot 0's flags (the struct has no holes)
    if (s < slots) {
      int rc = flag_alloc(&p->f.req[s]);
      if (rc == DH_OK) rc = flag_alloc(&p->f.done[s]);
      if (rc == DH_OK) rc = flag_alloc(&p->f.stop[s]);
      if (rc != DH_OK) return rc;
    } else {
      p->f.req[s] = p->f.req[0];
      p->f.done[s] = p->f.done[0];
      p->f.stop[s] = p->f.stop[0];
    }
  }
  const size_t log_bytes = sizeof(unsigned long long) * 2 * PROXY_LOG * PROXY_MAX_SLOTS;
  DH_HIP(hipMalloc((void **)&p->log, log_bytes));
  DH_HIP(hipMemset(p->log, 0, log_bytes));
  DH_HIP(hipDeviceSynchronize());
  *proxy_out = p;
  return DH_OK;
}

extern "C" int dh_comm_proxy_launch(void *proxy, int64_t duration_ns, int64_t limit_ns, void *stream) {
  using namespace dh;
  CommProxy *p = (CommProxy *)proxy;
  DH_CHECK(p != nullptr, "null proxy");
  DH_CHECK(!p->running, "the previous launch of this proxy has not been told to stop (dh_comm_proxy_stop)");
  DH_CHECK(duration_ns >= 0 && duration_ns <= 100000000ll, "duration of %lld ns outside [0, 0.1 s]", (long long)duration_ns);
  DH_CHECK(limit_ns >= 1000000ll && limit_ns <= 10000000000ll, "limit of %lld ns outside [1 ms, 10 s]", (long long)limit_ns);
  ++p->launch_no;
  hipLaunchKernelGGL(comm_proxy_kernel, dim3((unsigned)p->slots), dim3(64), 0, (hipStream_t)stream, p->f, p->log,
                     p->launch_no, (unsigned long long)(duration_ns / 10), (unsigned long long)(limit_ns / 10));
  DH_LAUNCH_CHECK();
  p->running = true;
  return DH_OK;
}

extern "C" int dh_comm_proxy_post(void *proxy, int slot, void *stream) {
  using namespace dh;
  CommProxy *p = (CommProxy *)proxy;
  const int rc = proxy_check(p, slot);
  if (rc != DH_OK) return rc;
  DH_CHECK(p->running, "no launch of this proxy is running");
  ++p->posted[slot];
  DH_HIP(hipStreamWriteValue32((hipStream_t)stream, p->f.req[slot], p->posted[slot], 0));
  return DH_OK;
}

extern "C" int dh_comm_proxy_wait(void *proxy, int slot, void *stream) {
  using namespace dh;
  CommProxy *p = (CommProxy *)proxy;
  const int rc = proxy_check(p, slot);
  if (rc != DH_OK) return rc;
  DH_HIP(hipStreamWaitValue32((hipStream_t)stream, p->f.done[slot], p->posted[slot], hipStreamWaitValueGte, 0xffffffffu));
  return DH_OK;
}

extern "C" int dh_comm_proxy_stop(void *proxy, const void *const *streams) {
  using namespace dh;
  CommProxy *p = (CommProxy *)proxy;
  DH_CHECK(p != nullptr && streams != nullptr, "null pointer");
  DH_CHECK(p->running, "no launch of this proxy is running");
  for (int s = 0; s < p->slots; ++s)
    DH_HIP(hipStreamWriteValue32((hipStream_t)streams[s], p->f.stop[s], p->launch_no, 0));
  p->running = false;
  return DH_OK;
}

extern "C" int dh_comm_proxy_log(void *proxy, int slot, int64_t max_entries, int64_t *start_ns, int64_t *end_ns,
                                 int64_t *n_out) {
  using namespace dh;
  CommProxy *p = (CommProxy *)proxy;
  const int rc = proxy_check(p, slot);
  if (rc != DH_OK) return rc;
  DH_CHECK(start_ns && end_ns && n_out && max_entries >= 0, "bad argument");
  std::vector<unsigned long long> h(2 * PROXY_LOG);
  DH_HIP(hipMemcpy(h.data(), p->log + (size_t)slot * PROXY_LOG * 2, sizeof(unsigned long long) * 2 * PROXY_LOG,
                   hipMemcpyDeviceToHost));
  int64_t n = 0;
  for (int k = 0; k < PROXY_LOG && n < max_entries; ++k) {
    if (h[2 * k + 1] == 0) break;
    start_ns[n] = (int64_t)h[2 * k] * 10;
    end_ns[n] = (int64_t)h[2 * k + 1] * 10;
    ++n;
  }
  *n_out = n;
  DH_HIP(hipMemset(p->log + (size_t)slot * PROXY_LOG * 2, 0, sizeof(unsigned long long) * 2 * PROXY_LOG));
  return DH_OK;
}

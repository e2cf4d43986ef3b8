// Shared device/host helpers for the gfx950 operator library.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>
#include <stddef.h>
#include "../../include/dhellam_hip.h"

namespace dh {

// ---- error reporting (thread-local message, integer status) ---------------
void set_error(const char *file, int line, const char *func, const char *fmt, ...);

#define DH_CHECK(cond, ...)                                              \
  do {                                                                   \
    if (!(cond)) {                                                       \
      ::dh::set_error(__FILE__, __LINE__, __func__, __VA_ARGS__);        \
      return DH_ERR_INVALID;                                             \
    }                                                                    \
  } while (0)

#define DH_HIP(call)                                                     \
  do {                                                                   \
    hipError_t e_ = (call);                                              \
    if (e_ != hipSuccess) {                                              \
      ::dh::set_error(__FILE__, __LINE__, __func__, "HIP error: %s",     \
                      hipGetErrorString(e_));                            \
      return DH_ERR_HIP;                                                 \
    }                                                                    \
  } while (0)

#define DH_LAUNCH_CHECK() DH_HIP(hipGetLastError())

// Raises a kernel's dynamic LDS limit once per (kernel, device): the attribute belongs to that pair, so the guard
// is one bit per device, set by whichever thread gets there first (setting it twice is harmless).  Use inside a
// function or function template that launches exactly this kernel; pass the kernel's address in parentheses.
#define DH_MAX_DYNAMIC_LDS_PER_DEVICE(kernel_addr, bytes)                                          \
  do {                                                                                             \
    static std::atomic<uint64_t> dh_attr_done_{0};                                                 \
    int dh_dev_ = 0;                                                                               \
    DH_HIP(hipGetDevice(&dh_dev_));                                                                \
    const uint64_t dh_bit_ = 1ull << (dh_dev_ & 63);                                               \
    if (!(dh_attr_done_.load(std::memory_order_acquire) & dh_bit_)) {                              \
      DH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel_addr),                      \
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes)));       \
      dh_attr_done_.fetch_or(dh_bit_, std::memory_order_release);                                  \
    }                                                                                              \
  } while (0)

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- scalar types -----------------------------------------------------------
using bf16_t = __bf16;
using f16_t = _Float16;

template <typename T> __device__ __forceinline__ float to_f(T v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T from_f(float v) { return static_cast<T>(v); }

// 16-byte vector of T, loaded/stored as one global transaction per lane.
template <typename T> struct alignas(16) Vec {
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

template <typename T> __device__ __forceinline__ Vec<T> ldg(const T *p) {
  return *reinterpret_cast<const Vec<T> *>(p);
}
template <typename T> __device__ __forceinline__ void stg(T *p, const Vec<T> &x) {
  *reinterpret_cast<Vec<T> *>(p) = x;
}

// Streaming variants for data touched once per kernel.  With NT the access carries the
// non-temporal hint: such lines do not displace reusable ones in L2 and the HBM rate of a pure
// streaming kernel rises by 10-30 % once its working set exceeds the 256 MB last-level cache;
// below that size the hint loses the cache hits a consumer kernel would get, so callers pass
// NT = stream_hint(bytes touched).
typedef uint32_t dh_u32x4 __attribute__((ext_vector_type(4)));
template <bool NT, typename T> __device__ __forceinline__ Vec<T> ldg_s(const T *p) {
  if constexpr (NT) {
    const dh_u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const dh_u32x4 *>(p));
    return __builtin_bit_cast(Vec<T>, r);
  } else {
    return ldg(p);
  }
}
template <bool NT, typename T> __device__ __forceinline__ void stg_s(T *p, const Vec<T> &x) {
  if constexpr (NT) {
    __builtin_nontemporal_store(__builtin_bit_cast(dh_u32x4, x), reinterpret_cast<dh_u32x4 *>(p));
  } else {
    stg(p, x);
  }
}
#ifndef DH_STREAM_HINT_BYTES
#define DH_STREAM_HINT_BYTES (256ll << 20)
#endif
static inline bool stream_hint(int64_t bytes_touched) { return bytes_touched > DH_STREAM_HINT_BYTES; }

// ---- wave64 reductions --------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Sum over a 256-thread block (4 waves); `red` is 4 floats of LDS per value.
__device__ __forceinline__ float block256_sum(float v, float *red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6;
  __syncthreads();  // protect `red` from the previous use
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// Sum over a block of BT threads (BT / 64 waves, BT in {256, 1024}); `red` holds BT / 64 floats.
template <int BT> __device__ __forceinline__ float block_sum(float v, float *red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6;
  __syncthreads();  // protect `red` from the previous use
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < BT / 64; ++i) t += red[i];
  return t;
}

// Dispatch a callable templated on the element type.
#define DH_DISPATCH_DTYPE(dtype, ...)                                    \
  switch (dtype) {                                                       \
    case DH_F32: { using T = float; __VA_ARGS__; } break;                \
    case DH_BF16: { using T = ::dh::bf16_t; __VA_ARGS__; } break;        \
    case DH_F16: { using T = ::dh::f16_t; __VA_ARGS__; } break;          \
    default:                                                             \
      ::dh::set_error(__FILE__, __LINE__, __func__, "unknown dtype %d", (int)(dtype)); \
      return DH_ERR_INVALID;                                             \
  }

static inline size_t dtype_size(int dtype) { return dtype == DH_F32 ? 4 : 2; }

}  // namespace dh

// Rotary position embedding (rotate-half) on q and k in the token-major
// [tokens, heads, d] layout the attention kernels consume.
//
// HBM-bound.  A lane owns one 16-byte chunk of the first half of the head
// dimension and the matching chunk of the second half, computes the chunk's
// cos/sin once (fp32 angle = pos * inv_freq[j]) and reuses them across the
// heads it walks, so the transcendental cost is amortised over hq + hk heads.
#include "common.h"

namespace dh {

template <typename T>
__global__ void __launch_bounds__(256)
rope_kernel(const T *__restrict__ q, const T *__restrict__ k, T *__restrict__ qo, T *__restrict__ ko,
            const float *__restrict__ inv_freq, const int32_t *__restrict__ positions, int64_t tokens, int hq,
            int hk, int d, int64_t q_stride, int64_t k_stride, int64_t qo_stride, int64_t ko_stride,
            int64_t seq_len, int hsplit, float sign) {
  constexpr int N = Vec<T>::N;
  const int half = d / 2;
  const int chunks = half / N;
  const int heads = hq + hk;
  const int hper = (heads + hsplit - 1) / hsplit;
  const int64_t nitems = tokens * hsplit * chunks;
  for (int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x; it < nitems; it += (int64_t)gridDim.x * 256) {
    const int c = (int)(it % chunks);
    const int64_t r = it / chunks;
    const int hs = (int)(r % hsplit);
    const int64_t t = r / hsplit;
    int64_t pos;
    if (positions) pos = positions[t];
    else pos = seq_len > 0 ? t % seq_len : t;
    float cs[N], sn[N];
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float ang = (float)pos * inv_freq[c * N + j];
      sincosf(ang, &sn[j], &cs[j]);
      sn[j] *= sign;
    }
    const int h0 = hs * hper;
    const int h1 = h0 + hper < heads ? h0 + hper : heads;
    for (int h = h0; h < h1; ++h) {
      const T *src;
      T *dst;
      if (h < hq) {
        src = q + t * q_stride + (int64_t)h * d;
        dst = qo + t * qo_stride + (int64_t)h * d;
      } else {
        src = k + t * k_stride + (int64_t)(h - hq) * d;
        dst = ko + t * ko_stride + (int64_t)(h - hq) * d;
      }
      const Vec<T> lo = ldg(src + c * N);
      const Vec<T> hi = ldg(src + half + c * N);
      Vec<T> olo, ohi;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const float a = to_f(lo.v[j]), b = to_f(hi.v[j]);
        olo.v[j] = from_f<T>(a * cs[j] - b * sn[j]);
        ohi.v[j] = from_f<T>(b * cs[j] + a * sn[j]);
      }
      stg(dst + c * N, olo);
      stg(dst + half + c * N, ohi);
    }
  }
}

}  // namespace dh

extern "C" int dh_rope(const void *q, const void *k, void *q_out, void *k_out, const float *inv_freq,
                       const int32_t *positions, int64_t tokens, int hq, int hk, int d, int64_t q_stride,
                       int64_t k_stride, int64_t qo_stride, int64_t ko_stride, int64_t seq_len, int backward,
                       int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(tokens >= 0 && hq >= 0 && hk >= 0 && d > 0, "bad shape tokens=%lld hq=%d hk=%d d=%d", (long long)tokens,
           hq, hk, d);
  if (tokens == 0 || hq + hk == 0) return DH_OK;
  DH_CHECK(inv_freq, "inv_freq is null");
  DH_CHECK(hq == 0 || (q && q_out), "q/q_out null with hq > 0");
  DH_CHECK(hk == 0 || (k && k_out), "k/k_out null with hk > 0");
  const int n = 16 / (int)dtype_size(dtype);
  DH_CHECK(d % (2 * n) == 0, "head dim %d must be a multiple of %d for this dtype", d, 2 * n);
  DH_CHECK(q_stride % n == 0 && k_stride % n == 0 && qo_stride % n == 0 && ko_stride % n == 0,
           "token strides must keep rows 16-byte aligned");
  DH_CHECK((!q || aligned16(q)) && (!k || aligned16(k)) && (!q_out || aligned16(q_out)) &&
               (!k_out || aligned16(k_out)),
           "q/k pointers must be 16-byte aligned");
  const int chunks = d / 2 / n;
  const int heads = hq + hk;
  // Split the heads over several lanes while the grid is too small to fill the chip.
  int hsplit = 1;
  while (hsplit < heads && tokens * chunks * hsplit < 256ll * 256 * 2) ++hsplit;
  const int64_t nitems = tokens * hsplit * chunks;
  int64_t blocks = cdiv(nitems, 256);
  if (blocks > 256 * 32) blocks = 256 * 32;
  const float sign = backward ? -1.0f : 1.0f;
  DH_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((rope_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const T *)q,
                       (const T *)k, (T *)q_out, (T *)k_out, inv_freq, positions, tokens, hq, hk, d, q_stride,
                       k_stride, qo_stride, ko_stride, seq_len, hsplit, sign);
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

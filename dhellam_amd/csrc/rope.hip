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
    // Heads are handled in groups of up to HG with all loads of a group issued first; the first group's loads go
    // out before the cos/sin evaluation (a few hundred instructions), which then runs in their shadow.
    constexpr int HG = 4;
    const int h0 = hs * hper;
    const int h1 = h0 + hper < heads ? h0 + hper : heads;
    Vec<T> lo[HG], hi[HG];
    auto src_of = [&](int h) {
      return h < hq ? q + t * q_stride + (int64_t)h * d : k + t * k_stride + (int64_t)(h - hq) * d;
    };
    auto dst_of = [&](int h) {
      return h < hq ? qo + t * qo_stride + (int64_t)h * d : ko + t * ko_stride + (int64_t)(h - hq) * d;
    };
    auto load_group = [&](int hb) {
#pragma unroll
      for (int g = 0; g < HG; ++g)
        if (hb + g < h1) {
          const T *src = src_of(hb + g);
          lo[g] = ldg(src + c * N);
          hi[g] = ldg(src + half + c * N);
        }
    };
    load_group(h0);
    float cs[N], sn[N];
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float ang = (float)pos * inv_freq[c * N + j];
      if (sizeof(T) == 4) {
        sincosf(ang, &sn[j], &cs[j]);
      } else {
        // 16-bit results: the hardware's sin / cos (argument in revolutions) after an exact reduction of the fp32
        // angle: ang / 2pi as a two-term product whose rounding error is recovered with an fma, so the fraction
        // of a revolution is good to ~1e-7 for angles of 1e5 rad; the routine's own error (~1e-6) is a thousand
        // times below the rounding of the result.
        const float c_hi = 0.15915494f, c_lo = 6.4206382e-9f;   // 1 / 2pi = c_hi + c_lo
        float r_hi = ang * c_hi;
        asm volatile("" : "+v"(r_hi));     // opaque to the compiler, which otherwise folds fma(a, b, -(a * b)) to zero
        const float r_lo = fmaf(ang, c_lo, fmaf(ang, c_hi, -r_hi));   // that fma recovers the product's rounding error
        const float rev = (r_hi - floorf(r_hi)) + r_lo;
        sn[j] = __builtin_amdgcn_sinf(rev);
        cs[j] = __builtin_amdgcn_cosf(rev);
      }
      sn[j] *= sign;
    }
    for (int hb = h0; hb < h1; hb += HG) {
      if (hb != h0) load_group(hb);
#pragma unroll
      for (int g = 0; g < HG; ++g)
        if (hb + g < h1) {
          Vec<T> olo, ohi;
#pragma unroll
          for (int j = 0; j < N; ++j) {
            const float a = to_f(lo[g].v[j]), b = to_f(hi[g].v[j]);
            olo.v[j] = from_f<T>(a * cs[j] - b * sn[j]);
            ohi.v[j] = from_f<T>(b * cs[j] + a * sn[j]);
          }
          T *dst = dst_of(hb + g);
          stg(dst + c * N, olo);
          stg(dst + half + c * N, ohi);
        }
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
  // (splitting further costs more than it gives: every lane of a split evaluates the chunk's cos / sin again;
  // 4096 tokens x 9 heads: 5.8 us with this bound, 6.9 / 7.6 us with twice / four times as many lanes)
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

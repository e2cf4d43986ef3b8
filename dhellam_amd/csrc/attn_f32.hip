// fp32 attention forward/backward without matrix cores.
//
// The fp32 path exists for the small full-precision parity configuration
// (hidden 1024, 16 heads x 64, seq 512); it is written for clarity and exact
// fp32 arithmetic, not speed.  One workgroup of 128 threads owns one query row
// (forward, dQ) or one key/value row (dK/dV) and walks the other sequence in
// chunks of 128: each thread scores one row of the chunk, the probabilities go
// through LDS, and each thread then accumulates the output columns it owns.
// Accumulation order is fixed, so results are deterministic.
#include "common.h"

namespace dh {

constexpr int F32_NT = 128;     // threads per block = rows per chunk
constexpr int F32_MAXC = 2;     // columns per thread (d <= 256)

__device__ __forceinline__ float block128_reduce(float v, float *red, bool is_max) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float u = __shfl_xor(v, o, 64);
    v = is_max ? fmaxf(v, u) : v + u;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return is_max ? fmaxf(red[0], red[1]) : red[0] + red[1];
}

__device__ __forceinline__ float dot_row(const float *a_lds, const float *__restrict__ b, int d) {
  float s = 0.f;
  for (int i = 0; i < d; i += 4) {
    const float4 x = *reinterpret_cast<const float4 *>(b + i);
    s += a_lds[i] * x.x + a_lds[i + 1] * x.y + a_lds[i + 2] * x.z + a_lds[i + 3] * x.w;
  }
  return s;
}

__global__ void __launch_bounds__(F32_NT)
attn_fwd_f32_kernel(const float *__restrict__ q, const float *__restrict__ k, const float *__restrict__ v,
                    float *__restrict__ out, float *__restrict__ lse, const int32_t *__restrict__ cu_q,
                    const int32_t *__restrict__ cu_k, int max_sq, int hq, int hk, int d, int64_t q_stride,
                    int64_t k_stride, int64_t v_stride, int64_t o_stride, float scale, int causal) {
  __shared__ float sq_row[256];
  __shared__ float sp[F32_NT];
  __shared__ float red[2];
  const int b = blockIdx.z, h = blockIdx.y, i = blockIdx.x;
  const int q0 = cu_q[b], sq = cu_q[b + 1] - q0;
  const int k0 = cu_k[b], sk = cu_k[b + 1] - k0;
  if (i >= sq) return;
  const int hkv = h / (hq / hk);
  const int tid = threadIdx.x;
  const float *qr = q + (int64_t)(q0 + i) * q_stride + (int64_t)h * d;
  for (int c = tid; c < d; c += F32_NT) sq_row[c] = qr[c];
  __syncthreads();
  const int kend = causal ? (i + 1 < sk ? i + 1 : sk) : sk;
  float m_run = -INFINITY, l_run = 0.f, acc[F32_MAXC] = {0.f, 0.f};
  for (int j0 = 0; j0 < kend; j0 += F32_NT) {
    const int j = j0 + tid;
    float s = -INFINITY;
    if (j < kend) s = scale * dot_row(sq_row, k + (int64_t)(k0 + j) * k_stride + (int64_t)hkv * d, d);
    const float m_new = fmaxf(m_run, block128_reduce(s, red, true));
    const float pj = j < kend ? expf(s - m_new) : 0.f;
    const float alpha = expf(m_run - m_new);  // 0 on the first chunk (m_run = -inf)
    const float psum = block128_reduce(pj, red, false);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    sp[tid] = pj;
    __syncthreads();
    const int cnt = kend - j0 < F32_NT ? kend - j0 : F32_NT;
#pragma unroll
    for (int ci = 0; ci < F32_MAXC; ++ci) {
      const int c = tid + ci * F32_NT;
      if (c < d) {
        float a = acc[ci] * alpha;
        const float *vp = v + (int64_t)(k0 + j0) * v_stride + (int64_t)hkv * d + c;
        for (int jj = 0; jj < cnt; ++jj) a += sp[jj] * vp[(int64_t)jj * v_stride];
        acc[ci] = a;
      }
    }
    __syncthreads();
  }
  float *orow = out + (int64_t)(q0 + i) * o_stride + (int64_t)h * d;
  const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
#pragma unroll
  for (int ci = 0; ci < F32_MAXC; ++ci) {
    const int c = tid + ci * F32_NT;
    if (c < d) orow[c] = acc[ci] * inv;
  }
  if (tid == 0) lse[((int64_t)b * hq + h) * max_sq + i] = l_run > 0.f ? m_run + logf(l_run) : -INFINITY;
}

// dQ: one block per query row.
__global__ void __launch_bounds__(F32_NT)
attn_bwd_dq_f32_kernel(const float *__restrict__ dout, const float *__restrict__ q, const float *__restrict__ k,
                       const float *__restrict__ v, const float *__restrict__ lse, const float *__restrict__ delta,
                       float *__restrict__ dq, const int32_t *__restrict__ cu_q, const int32_t *__restrict__ cu_k,
                       int max_sq, int hq, int hk, int d, int64_t q_stride, int64_t k_stride, int64_t v_stride,
                       int64_t do_stride, int64_t dq_stride, float scale, int causal, int accumulate) {
  __shared__ float sq_row[256], sdo_row[256];
  __shared__ float sds[F32_NT];
  const int b = blockIdx.z, h = blockIdx.y, i = blockIdx.x;
  const int q0 = cu_q[b], sq = cu_q[b + 1] - q0;
  const int k0 = cu_k[b], sk = cu_k[b + 1] - k0;
  if (i >= sq) return;
  const int hkv = h / (hq / hk);
  const int tid = threadIdx.x;
  const float *qr = q + (int64_t)(q0 + i) * q_stride + (int64_t)h * d;
  const float *dor = dout + (int64_t)(q0 + i) * do_stride + (int64_t)h * d;
  for (int c = tid; c < d; c += F32_NT) {
    sq_row[c] = qr[c];
    sdo_row[c] = dor[c];
  }
  __syncthreads();
  const float li = lse[((int64_t)b * hq + h) * max_sq + i];
  const float di = delta[((int64_t)b * hq + h) * max_sq + i];
  const int kend = causal ? (i + 1 < sk ? i + 1 : sk) : sk;
  float acc[F32_MAXC] = {0.f, 0.f};
  for (int j0 = 0; j0 < kend; j0 += F32_NT) {
    const int j = j0 + tid;
    float ds = 0.f;
    if (j < kend) {
      const float s = scale * dot_row(sq_row, k + (int64_t)(k0 + j) * k_stride + (int64_t)hkv * d, d);
      const float pj = expf(s - li);
      const float dp = dot_row(sdo_row, v + (int64_t)(k0 + j) * v_stride + (int64_t)hkv * d, d);
      ds = pj * (dp - di);
    }
    sds[tid] = ds;
    __syncthreads();
    const int cnt = kend - j0 < F32_NT ? kend - j0 : F32_NT;
#pragma unroll
    for (int ci = 0; ci < F32_MAXC; ++ci) {
      const int c = tid + ci * F32_NT;
      if (c < d) {
        float a = acc[ci];
        const float *kp = k + (int64_t)(k0 + j0) * k_stride + (int64_t)hkv * d + c;
        for (int jj = 0; jj < cnt; ++jj) a += sds[jj] * kp[(int64_t)jj * k_stride];
        acc[ci] = a;
      }
    }
    __syncthreads();
  }
  float *dqr = dq + (int64_t)(q0 + i) * dq_stride + (int64_t)h * d;
#pragma unroll
  for (int ci = 0; ci < F32_MAXC; ++ci) {
    const int c = tid + ci * F32_NT;
    if (c < d) dqr[c] = accumulate ? dqr[c] + acc[ci] * scale : acc[ci] * scale;
  }
}

// dK, dV: one block per key/value row; walks the query heads of its group and the
// query rows that attend to it.
__global__ void __launch_bounds__(F32_NT)
attn_bwd_dkv_f32_kernel(const float *__restrict__ dout, const float *__restrict__ q, const float *__restrict__ k,
                        const float *__restrict__ v, const float *__restrict__ lse,
                        const float *__restrict__ delta, float *__restrict__ dk, float *__restrict__ dv,
                        const int32_t *__restrict__ cu_q, const int32_t *__restrict__ cu_k, int max_sq, int hq,
                        int hk, int d, int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t do_stride,
                        int64_t dk_stride, int64_t dv_stride, float scale, int causal) {
  __shared__ float sk_row[256], sv_row[256];
  __shared__ float sp[F32_NT], sds[F32_NT];
  const int b = blockIdx.z, hkv = blockIdx.y, j = blockIdx.x;
  const int q0 = cu_q[b], sq = cu_q[b + 1] - q0;
  const int k0 = cu_k[b], sk = cu_k[b + 1] - k0;
  if (j >= sk) return;
  const int tid = threadIdx.x;
  const int ratio = hq / hk;
  const float *kr = k + (int64_t)(k0 + j) * k_stride + (int64_t)hkv * d;
  const float *vr = v + (int64_t)(k0 + j) * v_stride + (int64_t)hkv * d;
  for (int c = tid; c < d; c += F32_NT) {
    sk_row[c] = kr[c];
    sv_row[c] = vr[c];
  }
  __syncthreads();
  const int ibeg = causal ? j : 0;
  float ak[F32_MAXC] = {0.f, 0.f}, av[F32_MAXC] = {0.f, 0.f};
  for (int g = 0; g < ratio; ++g) {
    const int h = hkv * ratio + g;
    for (int i0 = ibeg; i0 < sq; i0 += F32_NT) {
      const int i = i0 + tid;
      float pj = 0.f, ds = 0.f;
      if (i < sq) {
        const float s = scale * dot_row(sk_row, q + (int64_t)(q0 + i) * q_stride + (int64_t)h * d, d);
        pj = expf(s - lse[((int64_t)b * hq + h) * max_sq + i]);
        const float dp = dot_row(sv_row, dout + (int64_t)(q0 + i) * do_stride + (int64_t)h * d, d);
        ds = pj * (dp - delta[((int64_t)b * hq + h) * max_sq + i]);
      }
      sp[tid] = pj;
      sds[tid] = ds;
      __syncthreads();
      const int cnt = sq - i0 < F32_NT ? sq - i0 : F32_NT;
#pragma unroll
      for (int ci = 0; ci < F32_MAXC; ++ci) {
        const int c = tid + ci * F32_NT;
        if (c < d) {
          float a1 = ak[ci], a2 = av[ci];
          const float *qp = q + (int64_t)(q0 + i0) * q_stride + (int64_t)h * d + c;
          const float *dp_ = dout + (int64_t)(q0 + i0) * do_stride + (int64_t)h * d + c;
          for (int ii = 0; ii < cnt; ++ii) {
            a1 += sds[ii] * qp[(int64_t)ii * q_stride];
            a2 += sp[ii] * dp_[(int64_t)ii * do_stride];
          }
          ak[ci] = a1;
          av[ci] = a2;
        }
      }
      __syncthreads();
    }
  }
  float *dkr = dk + (int64_t)(k0 + j) * dk_stride + (int64_t)hkv * d;
  float *dvr = dv + (int64_t)(k0 + j) * dv_stride + (int64_t)hkv * d;
#pragma unroll
  for (int ci = 0; ci < F32_MAXC; ++ci) {
    const int c = tid + ci * F32_NT;
    if (c < d) {
      dkr[c] = ak[ci] * scale;
      dvr[c] = av[ci];
    }
  }
}

int attn_fwd_f32(const void *q, const void *k, const void *v, void *out, float *lse, const int32_t *cu_q,
                 const int32_t *cu_k, int batch, int max_sq, int max_sk, int hq, int hk, int d, int64_t q_stride,
                 int64_t k_stride, int64_t v_stride, int64_t o_stride, float scale, int causal, hipStream_t st) {
  DH_CHECK(q_stride % 4 == 0 && k_stride % 4 == 0 && v_stride % 4 == 0 && aligned16(q) && aligned16(k) && aligned16(v),
           "fp32 attention needs 16-byte aligned rows");
  hipLaunchKernelGGL(attn_fwd_f32_kernel, dim3((unsigned)max_sq, (unsigned)hq, (unsigned)batch), dim3(F32_NT), 0, st,
                     (const float *)q, (const float *)k, (const float *)v, (float *)out, lse, cu_q, cu_k, max_sq, hq,
                     hk, d, q_stride, k_stride, v_stride, o_stride, scale, causal);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

int attn_bwd_f32(const void *dout, const void *q, const void *k, const void *v, const float *lse, const float *delta,
                 void *dq, void *dk, void *dv, const int32_t *cu_q, const int32_t *cu_k, int batch, int max_sq,
                 int max_sk, int hq, int hk, int d, int64_t q_stride, int64_t k_stride, int64_t v_stride,
                 int64_t do_stride, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride, float scale, int causal,
                 int dq_accumulate, hipStream_t st) {
  DH_CHECK(q_stride % 4 == 0 && k_stride % 4 == 0 && v_stride % 4 == 0 && do_stride % 4 == 0 && aligned16(q) &&
               aligned16(k) && aligned16(v) && aligned16(dout),
           "fp32 attention needs 16-byte aligned rows");
  if (max_sq > 0)
    hipLaunchKernelGGL(attn_bwd_dq_f32_kernel, dim3((unsigned)max_sq, (unsigned)hq, (unsigned)batch), dim3(F32_NT), 0,
                       st, (const float *)dout, (const float *)q, (const float *)k, (const float *)v, lse, delta,
                       (float *)dq, cu_q, cu_k, max_sq, hq, hk, d, q_stride, k_stride, v_stride, do_stride, dq_stride,
                       scale, causal, dq_accumulate);
  if (max_sk > 0)
    hipLaunchKernelGGL(attn_bwd_dkv_f32_kernel, dim3((unsigned)max_sk, (unsigned)hk, (unsigned)batch), dim3(F32_NT),
                       0, st, (const float *)dout, (const float *)q, (const float *)k, (const float *)v, lse, delta,
                       (float *)dk, (float *)dv, cu_q, cu_k, max_sq, hq, hk, d, q_stride, k_stride, v_stride,
                       do_stride, dk_stride, dv_stride, scale, causal);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

}  // namespace dh

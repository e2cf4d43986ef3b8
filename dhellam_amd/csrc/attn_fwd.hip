// Causal / non-causal GQA flash-attention forward on bf16/fp16 MFMA (gfx950).
//
// One workgroup = NW wavefronts, each owning 32 query rows of one head; K/V
// tiles of 64 rows are staged in LDS (two stages, one barrier per tile) and
// shared by the wavefronts.  Per tile a wavefront computes S^T = K Q^T (Q
// fragments live in registers for the whole kernel), so that every lane holds
// 32 scores of ONE query row: the online-softmax row reductions are in-lane
// plus a single exchange with lane^32.  P^T never leaves registers: its
// accumulator layout is fed back as the B operand of O^T += V^T P^T, with the
// matching V^T fragments produced by LDS transpose reads from the row-major V
// tile.  fp32 scores are scaled inside the exp2 argument (one FMA), the running
// output is rescaled only when some row's maximum actually moved.
#include "mma.h"

namespace dh {

struct AttnFwdParams {
  const void *q, *k, *v;
  void *o;
  float *lse;
  const int32_t *cu_q, *cu_k;
  int max_sq, hq, hk;
  int64_t q_stride, k_stride, v_stride, o_stride;
  float scale, scale_log2;
  int causal;
};

template <typename T, int D, int NW>
__global__ void __launch_bounds__(64 * NW) attn_fwd_kernel(const AttnFwdParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int BM = 32 * NW, BN = 64, NT = 64 * NW;
  constexpr int KS = D + 8;    // K tile row stride (elements): 16 B pad, conflict-free 16 B row reads
  constexpr int VS = D + 32;   // V tile row stride: 64 B pad, conflict-free transpose reads
  constexpr int VPR = D / 8;   // 16-byte vectors per row
  constexpr int LPT = BN * VPR / NT;  // vectors per thread per tile
  static_assert(BN * VPR % NT == 0, "tile must divide over the block");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T *sK = reinterpret_cast<T *>(smem_raw);  // [2][BN*KS]
  T *sV = sK + 2 * BN * KS;                 // [2][BN*VS]

  const int b = blockIdx.z, h = blockIdx.y;
  const int mt = gridDim.x - 1 - blockIdx.x;  // heavy (late) causal tiles first
  const int q0 = p.cu_q[b], sq = p.cu_q[b + 1] - q0;
  const int k0 = p.cu_k[b], sk = p.cu_k[b + 1] - k0;
  const int m0 = mt * BM;
  if (m0 >= sq) return;
  const int hkv = h / (p.hq / p.hk);
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int c = lane & 31, hh = lane >> 5;
  const int wrow0 = m0 + w * 32;
  const int row_q = wrow0 + c;
  const int row_ld = row_q < sq ? row_q : sq - 1;

  const T *qp = reinterpret_cast<const T *>(p.q) + (int64_t)(q0 + row_ld) * p.q_stride + (int64_t)h * D;
  Frag Qf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) Qf[ks] = frag_ld<T>(qp + ks * 16 + 8 * hh);

  const T *kg = reinterpret_cast<const T *>(p.k) + (int64_t)k0 * p.k_stride + (int64_t)hkv * D;
  const T *vg = reinterpret_cast<const T *>(p.v) + (int64_t)k0 * p.v_stride + (int64_t)hkv * D;

  int nk_end = sk;
  if (p.causal && m0 + BM < nk_end) nk_end = m0 + BM;
  const int ntiles = (nk_end + BN - 1) / BN;

  floatx16 O[D / 32];
#pragma unroll
  for (int t = 0; t < D / 32; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) O[t][v] = 0.f;
  float m_run = -1e30f, l_run = 0.f;

  uint4 rk[LPT], rv[LPT];
  auto gload = [&](int n0) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int idx = tid + i * NT;
      const int r = idx / VPR, cv = idx % VPR;
      const int kr = n0 + r;
      if (kr < sk) {
        rk[i] = *reinterpret_cast<const uint4 *>(kg + (int64_t)kr * p.k_stride + cv * 8);
        rv[i] = *reinterpret_cast<const uint4 *>(vg + (int64_t)kr * p.v_stride + cv * 8);
      } else {
        rk[i] = make_uint4(0, 0, 0, 0);
        rv[i] = make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto sstore = [&](int st) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int idx = tid + i * NT;
      const int r = idx / VPR, cv = idx % VPR;
      *reinterpret_cast<uint4 *>(sK + st * BN * KS + r * KS + cv * 8) = rk[i];
      *reinterpret_cast<uint4 *>(sV + st * BN * VS + r * VS + cv * 8) = rv[i];
    }
  };

  if (ntiles > 0) {
    gload(0);
    sstore(0);
  }
  __syncthreads();

  for (int it = 0; it < ntiles; ++it) {
    const int n0 = it * BN;
    const int st = it & 1;
    if (it + 1 < ntiles) gload(n0 + BN);

    // A wavefront whose 32 rows all lie above this tile (causal) has nothing to do.
    const bool skip = p.causal && n0 > wrow0 + 31;
    if (!skip) {
      const T *tK = sK + st * BN * KS;
      const T *tV = sV + st * BN * VS;
      floatx16 S[2];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) S[nb][v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
          const Frag a = frag_ld<T>(tK + (nb * 32 + c) * KS + ks * 16 + 8 * hh);
          S[nb] = M::mma(a, Qf[ks], S[nb]);
        }
      }
      const bool need_mask = (p.causal && n0 + BN - 1 > wrow0) || (n0 + BN > sk);
      if (need_mask) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int kv = n0 + nb * 32 + acc_row(v, hh);
            if (kv >= sk || (p.causal && kv > row_q)) S[nb][v] = -INFINITY;
          }
      }
      float mx = S[0][0];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, S[nb][v]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      if (__any(m_new > m_run)) {
        const float alpha = fast_exp2((m_run - m_new) * p.scale_log2);
        l_run *= alpha;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) O[t][v] *= alpha;
      }
      m_run = m_new;
      const float mc = m_new * p.scale_log2;
      float ps = 0.f;
      Frag Pb[4];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        float pv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          pv[j] = fast_exp2(S[s >> 1][8 * (s & 1) + j] * p.scale_log2 - mc);
          ps += pv[j];
        }
        Pb[s] = frag_pack<T>(pv);
      }
      l_run += ps;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
#pragma unroll
        for (int t = 0; t < D / 32; ++t) {
          const Frag vf = frag_ld_tr<T>(tV, VS, 16 * s + 4 * hh, 16 * s + 8 + 4 * hh, 32 * t + 16 * ((lane >> 4) & 1), lane);
          O[t] = M::mma(vf, Pb[s], O[t]);
        }
      }
    }
    if (it + 1 < ntiles) sstore(st ^ 1);
    __syncthreads();
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if (row_q < sq) {
    T *op = reinterpret_cast<T *>(p.o) + (int64_t)(q0 + row_q) * p.o_stride + (int64_t)h * D;
#pragma unroll
    for (int t = 0; t < D / 32; ++t)
#pragma unroll
      for (int vb = 0; vb < 4; ++vb) {
        struct alignas(8) { T v[4]; } o4;
#pragma unroll
        for (int j = 0; j < 4; ++j) o4.v[j] = static_cast<T>(O[t][4 * vb + j] * inv);
        *reinterpret_cast<decltype(o4) *>(op + 32 * t + 8 * vb + 4 * hh) = o4;
      }
    if (hh == 0)
      p.lse[((int64_t)b * p.hq + h) * p.max_sq + row_q] = l_tot > 0.f ? m_run * p.scale + logf(l_tot) : -INFINITY;
  }
}

template <typename T, int D, int NW>
static int launch_attn_fwd(const AttnFwdParams &p, int batch, hipStream_t st) {
  constexpr int BM = 32 * NW, BN = 64;
  constexpr size_t smem = 2 * BN * ((D + 8) + (D + 32)) * sizeof(T);
  static bool attr_set = false;
  if (!attr_set) {
    DH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_fwd_kernel<T, D, NW>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    attr_set = true;
  }
  dim3 grid((unsigned)cdiv(p.max_sq, BM), (unsigned)p.hq, (unsigned)batch);
  hipLaunchKernelGGL((attn_fwd_kernel<T, D, NW>), grid, dim3(64 * NW), smem, st, p);
  return DH_OK;
}

int attn_fwd_f32(const void *q, const void *k, const void *v, void *out, float *lse, const int32_t *cu_q,
                 const int32_t *cu_k, int batch, int max_sq, int max_sk, int hq, int hk, int d, int64_t q_stride,
                 int64_t k_stride, int64_t v_stride, int64_t o_stride, float scale, int causal, hipStream_t st);

}  // namespace dh

extern "C" int dh_attn_fwd(const void *q, const void *k, const void *v, void *out, float *lse,
                           const int32_t *cu_seqlens_q, const int32_t *cu_seqlens_k, int batch, int max_seqlen_q,
                           int max_seqlen_k, int hq, int hk, int d, int64_t q_stride, int64_t k_stride,
                           int64_t v_stride, int64_t o_stride, float softmax_scale, int causal, int dtype,
                           void *stream) {
  using namespace dh;
  DH_CHECK(batch >= 0 && max_seqlen_q >= 0 && max_seqlen_k >= 0, "negative size");
  DH_CHECK(hq > 0 && hk > 0 && hq % hk == 0, "hq=%d must be a positive multiple of hk=%d", hq, hk);
  if (batch == 0 || max_seqlen_q == 0) return DH_OK;
  DH_CHECK(q && k && v && out && lse && cu_seqlens_q && cu_seqlens_k, "null pointer");
  DH_CHECK(q_stride >= (int64_t)hq * d && o_stride >= (int64_t)hq * d && k_stride >= (int64_t)hk * d &&
               v_stride >= (int64_t)hk * d,
           "token stride smaller than heads*d");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == DH_F32) {
    DH_CHECK(d > 0 && d <= 256 && d % 4 == 0, "fp32 attention needs d %% 4 == 0 and d <= 256 (got %d)", d);
    return attn_fwd_f32(q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k, batch, max_seqlen_q, max_seqlen_k, hq, hk, d,
                        q_stride, k_stride, v_stride, o_stride, softmax_scale, causal, st);
  }
  DH_CHECK(dtype == DH_BF16 || dtype == DH_F16, "unknown dtype %d", dtype);
  DH_CHECK(d == 64 || d == 128, "bf16/fp16 attention supports head dim 64 or 128 (got %d)", d);
  DH_CHECK(q_stride % 8 == 0 && k_stride % 8 == 0 && v_stride % 8 == 0 && o_stride % 4 == 0,
           "token strides must keep rows 16-byte aligned");
  DH_CHECK(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out), "q/k/v/out must be 16-byte aligned");
  AttnFwdParams p;
  p.q = q; p.k = k; p.v = v; p.o = out; p.lse = lse;
  p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k;
  p.max_sq = max_seqlen_q; p.hq = hq; p.hk = hk;
  p.q_stride = q_stride; p.k_stride = k_stride; p.v_stride = v_stride; p.o_stride = o_stride;
  p.scale = softmax_scale;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  p.causal = causal;
  // Few query tiles (small batch*heads) -> smaller workgroups so the grid still covers the chip.
  const int64_t blocks128 = cdiv(max_seqlen_q, 128) * hq * batch;
  const bool small = blocks128 < 2 * 256;
  int rc;
  if (dtype == DH_BF16) {
    if (d == 128) rc = small ? launch_attn_fwd<bf16_t, 128, 2>(p, batch, st) : launch_attn_fwd<bf16_t, 128, 4>(p, batch, st);
    else rc = small ? launch_attn_fwd<bf16_t, 64, 2>(p, batch, st) : launch_attn_fwd<bf16_t, 64, 4>(p, batch, st);
  } else {
    if (d == 128) rc = small ? launch_attn_fwd<f16_t, 128, 2>(p, batch, st) : launch_attn_fwd<f16_t, 128, 4>(p, batch, st);
    else rc = small ? launch_attn_fwd<f16_t, 64, 2>(p, batch, st) : launch_attn_fwd<f16_t, 64, 4>(p, batch, st);
  }
  if (rc != DH_OK) return rc;
  DH_LAUNCH_CHECK();
  return DH_OK;
}

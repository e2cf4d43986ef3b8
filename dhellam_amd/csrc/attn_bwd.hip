// Flash-attention backward on bf16/fp16 MFMA (gfx950), deterministic (no
// floating-point atomics).
//
// Three kernels:
//   delta   : delta_i = sum_d dO[i,d] * O[i,d]                      (streaming; head dim 64 only: the
//             head dim 128 dQ kernel forms delta in its prologue and runs first)
//   dK/dV   : a workgroup owns 64 key/value rows (K, V fragments stay in
//             registers for head dim 64, in LDS for head dim 128), walks the
//             query heads of its GQA group and the query tiles that attend to
//             it; S = Q K^T and dP = dO V^T are computed
//             with the key index on lanes so that P and dS feed dV^T += dO^T P
//             and dK^T += Q^T dS straight from their accumulators, with the
//             transposed Q / dO fragments coming from LDS transpose reads.
//             The GQA group sum happens in the accumulators; when the grid
//             would be too small the group is split over workgroups and a small
//             kernel adds the fp32 partials in a fixed order.
//   dQ      : a workgroup owns 32*NW query rows (Q, dO fragments in registers),
//             walks the key tiles; S^T, dP^T have the query index on lanes and
//             dS^T feeds dQ^T += K^T dS^T.
// Recomputing S and dP in both passes costs 7 matrix products instead of 5 but
// needs no fp32 dQ accumulator in memory and no atomics.
#include <atomic>

#include "mma.h"


namespace dh {

struct AttnBwdParams {
  const void *dout, *q, *k, *v;
  const void *out;           // forward output (d = 128: the dQ kernel forms delta from it)
  int64_t o_stride;
  const float *lse;
  float *delta;              // fp32 [batch][hq][max_sq]: rowsum(dO * O); written by the delta kernel, or (d = 128) by the dQ kernel
  float *ld2;                // fp32 [2][plane]: lse * log2(e), then delta, each [batch][hq][ld2_pitch] (d = 128 kernels)
  int64_t ld2_plane;         // elements between the two planes
  int ld2_pitch;             // max_sq rounded up to 32: every 32-row query tile of a head is one aligned 128-byte run
  void *dq, *dk, *dv;
  float *dk_part, *dv_part;  // fp32 [hsplit][total_k][hk][d] when hsplit > 1
  const int32_t *cu_q, *cu_k;
  int max_sq, hq, hk, hsplit;
  int64_t total_k;
  int64_t q_stride, k_stride, v_stride, do_stride, dq_stride, dk_stride, dv_stride;
  float scale, scale_log2;
  int causal;
  int dq_accumulate;         // dq += this call's gradient (read, add in fp32, round once) instead of dq =
  // dS = P * (dP - delta) kept for the dQ product (head dim 128, 16 bits, when the workspace allows): 2 KB blocks of
  // 32 keys x 32 query rows, block (b, h, query tile, key block); inside a block the 16-byte piece (s, hh, key)
  // holds the query rows 16 s + 8 u + 4 hh + x of that key (u = 0, 1; x = 0..3): what a lane of the dK/dV kernel
  // has in its packed dS fragment s.
  void *ds;
  int ds_nqt, ds_nkb;        // query tiles and key blocks (of 32) per (batch, head)
};

// ---- delta = rowsum(dO * O) ---------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
attn_delta_kernel(const T *__restrict__ dout, const T *__restrict__ out, float *__restrict__ delta,
                  const float *__restrict__ lse, float *__restrict__ ld2, int64_t ld2_plane, int ld2_pitch,
                  const int32_t *__restrict__ cu_q, int max_sq, int hq, int d, int lanes_per, int64_t do_stride,
                  int64_t o_stride) {
  constexpr int N = Vec<T>::N;
  const int b = blockIdx.y;
  const int q0 = cu_q[b], sq = cu_q[b + 1] - q0;
  const int per_block = 256 / lanes_per;
  const int sub = threadIdx.x / lanes_per, ln = threadIdx.x % lanes_per;
  const int nvec = d / N;
  const int rows = ld2 ? ((sq + 31) / 32) * 32 : sq;   // the side-by-side planes are written in whole 32-row tiles
  for (int64_t item = (int64_t)blockIdx.x * per_block + sub; item < (int64_t)rows * hq;
       item += (int64_t)gridDim.x * per_block) {
    const int i = (int)(item / hq), h = (int)(item % hq);
    if (i >= sq) {           // padding rows of the last tile: zeros, so that masked scores stay finite
      if (ln == 0) {
        const int64_t a2 = ((int64_t)b * hq + h) * ld2_pitch + i;
        ld2[a2] = 0.f;
        ld2[ld2_plane + a2] = 0.f;
      }
      continue;
    }
    float s = 0.f;
    for (int c = ln; c < nvec; c += lanes_per) {
      const Vec<T> a = ldg(dout + (int64_t)(q0 + i) * do_stride + (int64_t)h * d + c * N);
      const Vec<T> o = ldg(out + (int64_t)(q0 + i) * o_stride + (int64_t)h * d + c * N);
#pragma unroll
      for (int j = 0; j < N; ++j) s += to_f(a.v[j]) * to_f(o.v[j]);
    }
    for (int o = lanes_per >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    if (ln == 0) {
      const int64_t at = ((int64_t)b * hq + h) * max_sq + i;
      delta[at] = s;
      if (ld2) {             // the copy the d = 128 kernels stream: lse in exp2 units next to delta
        const int64_t a2 = ((int64_t)b * hq + h) * ld2_pitch + i;
        ld2[a2] = lse[at] * 1.4426950408889634f;
        ld2[ld2_plane + a2] = s;
      }
    }
  }
}

// ---- dK, dV ---------------------------------------------------------------------------------
template <typename T, int D, int NW>
__global__ void __launch_bounds__(64 * NW) attn_bwd_dkv_kernel(const AttnBwdParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int BN = 32 * NW, BM = 32, NT = 64 * NW;
  constexpr int QS = D + 16;  // row stride of the Q / dO tiles (row reads and transpose reads)
  constexpr int VPR = D / 8;
  constexpr int LPT = BM * VPR / NT;
  static_assert(BM * VPR % NT == 0, "tile must divide over the block");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T *sQ = reinterpret_cast<T *>(smem_raw);        // [2][BM*QS]
  T *sdO = sQ + 2 * BM * QS;                      // [2][BM*QS]
  float *sLse = reinterpret_cast<float *>(sdO + 2 * BM * QS);  // [2][BM]  (lse * log2e, +inf for rows >= sq)
  float *sDel = sLse + 2 * BM;                                 // [2][BM]

  const int b = blockIdx.z;
  const int hkv = blockIdx.y / p.hsplit, hs = blockIdx.y % p.hsplit;
  const int q0 = p.cu_q[b], sq = p.cu_q[b + 1] - q0;
  const int k0 = p.cu_k[b], sk = p.cu_k[b + 1] - k0;
  const int j0 = blockIdx.x * BN;  // causal: low tiles carry the most work and come first
  if (j0 >= sk) return;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int c = lane & 31, hh = lane >> 5;
  const int jw0 = j0 + 32 * w;
  const int jrow = jw0 + c;
  const int ratio = p.hq / p.hk;
  const int hper = ratio / p.hsplit;

  Frag Kf[D / 16], Vf[D / 16];
  {
    const int jl = jrow < sk ? jrow : sk - 1;
    const T *kp = reinterpret_cast<const T *>(p.k) + (int64_t)(k0 + jl) * p.k_stride + (int64_t)hkv * D;
    const T *vp = reinterpret_cast<const T *>(p.v) + (int64_t)(k0 + jl) * p.v_stride + (int64_t)hkv * D;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      Kf[ks] = frag_ld<T>(kp + ks * 16 + 8 * hh);
      Vf[ks] = frag_ld<T>(vp + ks * 16 + 8 * hh);
    }
  }
  floatx16 dKt[D / 32], dVt[D / 32];
#pragma unroll
  for (int t = 0; t < D / 32; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      dKt[t][v] = 0.f;
      dVt[t][v] = 0.f;
    }

  const int i_begin = p.causal ? (j0 / BM) * BM : 0;
  const int ntq = i_begin < sq ? (sq - i_begin + BM - 1) / BM : 0;
  const int nsteps = ntq * hper;

  uint4 rq[LPT], rdo[LPT];
  float rl = 0.f, rd = 0.f;
  auto gload = [&](int step) {
    const int g = step / ntq, ti = step % ntq;
    const int h = hkv * ratio + hs * hper + g;
    const int i0 = i_begin + ti * BM;
    const T *qg = reinterpret_cast<const T *>(p.q) + (int64_t)q0 * p.q_stride + (int64_t)h * D;
    const T *dg = reinterpret_cast<const T *>(p.dout) + (int64_t)q0 * p.do_stride + (int64_t)h * D;
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int idx = tid + i * NT;
      const int r = idx / VPR, cv = idx % VPR;
      const int ir = i0 + r;
      if (ir < sq) {
        rq[i] = *reinterpret_cast<const uint4 *>(qg + (int64_t)ir * p.q_stride + cv * 8);
        rdo[i] = *reinterpret_cast<const uint4 *>(dg + (int64_t)ir * p.do_stride + cv * 8);
      } else {
        rq[i] = make_uint4(0, 0, 0, 0);
        rdo[i] = make_uint4(0, 0, 0, 0);
      }
    }
    if (tid < BM) {
      const int ir = i0 + tid;
      if (ir < sq) {
        rl = p.lse[((int64_t)b * p.hq + h) * p.max_sq + ir] * 1.4426950408889634f;
        rd = p.delta[((int64_t)b * p.hq + h) * p.max_sq + ir];
      } else {
        rl = INFINITY;
        rd = 0.f;
      }
    }
  };
  auto sstore = [&](int st) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int idx = tid + i * NT;
      const int r = idx / VPR, cv = idx % VPR;
      *reinterpret_cast<uint4 *>(sQ + st * BM * QS + r * QS + cv * 8) = rq[i];
      *reinterpret_cast<uint4 *>(sdO + st * BM * QS + r * QS + cv * 8) = rdo[i];
    }
    if (tid < BM) {
      sLse[st * BM + tid] = rl;
      sDel[st * BM + tid] = rd;
    }
  };

  if (nsteps > 0) {
    gload(0);
    sstore(0);
  }
  __syncthreads();

  for (int step = 0; step < nsteps; ++step) {
    const int st = step & 1;
    if (step + 1 < nsteps) gload(step + 1);
    const int i0 = i_begin + (step % ntq) * BM;
    // causal: the whole 32-row query block lies above this wavefront's keys -> nothing to add
    const bool skip = p.causal && i0 + BM - 1 < jw0;
    if (!skip) {
      const T *tQ = sQ + st * BM * QS;
      const T *tdO = sdO + st * BM * QS;
      floatx16 S, dP;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        S[v] = 0.f;
        dP[v] = 0.f;
      }
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        const Frag aq = frag_ld<T>(tQ + c * QS + ks * 16 + 8 * hh);
        S = M::mma(aq, Kf[ks], S);
        const Frag ad = frag_ld<T>(tdO + c * QS + ks * 16 + 8 * hh);
        dP = M::mma(ad, Vf[ks], dP);
      }
      const bool need_mask = p.causal && i0 < jw0 + 31;
      float pv[16], dsv[16];
#pragma unroll
      for (int vb = 0; vb < 4; ++vb) {
        const float4 l4 = *reinterpret_cast<const float4 *>(sLse + st * BM + 8 * vb + 4 * hh);
        const float4 d4 = *reinterpret_cast<const float4 *>(sDel + st * BM + 8 * vb + 4 * hh);
        const float ls[4] = {l4.x, l4.y, l4.z, l4.w};
        const float dl[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int v = 4 * vb + e;
          float pe = fast_exp2(S[v] * p.scale_log2 - ls[e]);
          if (need_mask && jrow > i0 + acc_row(v, hh)) pe = 0.f;
          pv[v] = pe;
          dsv[v] = pe * (dP[v] - dl[e]);
        }
      }
      Frag Pb[2], dSb[2];
      Pb[0] = frag_pack<T>(pv);
      Pb[1] = frag_pack<T>(pv + 8);
      dSb[0] = frag_pack<T>(dsv);
      dSb[1] = frag_pack<T>(dsv + 8);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int t = 0; t < D / 32; ++t) {
          const int n0 = 32 * t + 16 * ((lane >> 4) & 1);
          const Frag ad = frag_ld_tr<T>(tdO, QS, 16 * s + 4 * hh, 16 * s + 8 + 4 * hh, n0, lane);
          dVt[t] = M::mma(ad, Pb[s], dVt[t]);
          const Frag aq = frag_ld_tr<T>(tQ, QS, 16 * s + 4 * hh, 16 * s + 8 + 4 * hh, n0, lane);
          dKt[t] = M::mma(aq, dSb[s], dKt[t]);
        }
      }
    }
    if (step + 1 < nsteps) sstore(st ^ 1);
    __syncthreads();
  }

  if (jrow < sk) {
    if (p.hsplit == 1) {
      T *dkp = reinterpret_cast<T *>(p.dk) + (int64_t)(k0 + jrow) * p.dk_stride + (int64_t)hkv * D;
      T *dvp = reinterpret_cast<T *>(p.dv) + (int64_t)(k0 + jrow) * p.dv_stride + (int64_t)hkv * D;
#pragma unroll
      for (int t = 0; t < D / 32; ++t)
#pragma unroll
        for (int vb = 0; vb < 4; ++vb) {
          struct alignas(8) { T v[4]; } a, bq;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            a.v[e] = static_cast<T>(dKt[t][4 * vb + e] * p.scale);
            bq.v[e] = static_cast<T>(dVt[t][4 * vb + e]);
          }
          *reinterpret_cast<decltype(a) *>(dkp + 32 * t + 8 * vb + 4 * hh) = a;
          *reinterpret_cast<decltype(bq) *>(dvp + 32 * t + 8 * vb + 4 * hh) = bq;
        }
    } else {
      const int64_t off = (((int64_t)hs * p.total_k + (k0 + jrow)) * p.hk + hkv) * D;
#pragma unroll
      for (int t = 0; t < D / 32; ++t)
#pragma unroll
        for (int vb = 0; vb < 4; ++vb) {
          *reinterpret_cast<float4 *>(p.dk_part + off + 32 * t + 8 * vb + 4 * hh) =
              make_float4(dKt[t][4 * vb] * p.scale, dKt[t][4 * vb + 1] * p.scale, dKt[t][4 * vb + 2] * p.scale,
                          dKt[t][4 * vb + 3] * p.scale);
          *reinterpret_cast<float4 *>(p.dv_part + off + 32 * t + 8 * vb + 4 * hh) =
              make_float4(dVt[t][4 * vb], dVt[t][4 * vb + 1], dVt[t][4 * vb + 2], dVt[t][4 * vb + 3]);
        }
    }
  }
}

// Sum of the head-split partials, in split order: part fp32 [hsplit][total_k][hk][d] -> dst (T, strided rows).
template <typename T>
__global__ void __launch_bounds__(256)
attn_bwd_gqa_sum_kernel(const float *__restrict__ dk_part, const float *__restrict__ dv_part, T *__restrict__ dk,
                        T *__restrict__ dv, int64_t total_k, int hk, int d, int hsplit, int64_t dk_stride,
                        int64_t dv_stride) {
  const int dv4 = d / 4;
  const int64_t nitems = total_k * hk * dv4;
  for (int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x; it < nitems; it += (int64_t)gridDim.x * 256) {
    const int cc = (int)(it % dv4);
    const int64_t r = it / dv4;
    const int h = (int)(r % hk);
    const int64_t j = r / hk;
    float4 a = make_float4(0, 0, 0, 0), bb = make_float4(0, 0, 0, 0);
    for (int s = 0; s < hsplit; ++s) {
      const int64_t off = (((int64_t)s * total_k + j) * hk + h) * d + cc * 4;
      const float4 x = *reinterpret_cast<const float4 *>(dk_part + off);
      const float4 y = *reinterpret_cast<const float4 *>(dv_part + off);
      a.x += x.x; a.y += x.y; a.z += x.z; a.w += x.w;
      bb.x += y.x; bb.y += y.y; bb.z += y.z; bb.w += y.w;
    }
    T *pk = dk + j * dk_stride + (int64_t)h * d + cc * 4;
    T *pv = dv + j * dv_stride + (int64_t)h * d + cc * 4;
    pk[0] = from_f<T>(a.x); pk[1] = from_f<T>(a.y); pk[2] = from_f<T>(a.z); pk[3] = from_f<T>(a.w);
    pv[0] = from_f<T>(bb.x); pv[1] = from_f<T>(bb.y); pv[2] = from_f<T>(bb.z); pv[3] = from_f<T>(bb.w);
  }
}

// ---- dQ ---------------------------------------------------------------------------------------
template <typename T, int D, int NW>
__global__ void __launch_bounds__(64 * NW) attn_bwd_dq_kernel(const AttnBwdParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int BM = 32 * NW, BN = 32, NT = 64 * NW;
  constexpr int KS = D + 16;  // K tile: row reads and transpose reads
  constexpr int VS = D + 8;   // V tile: row reads only
  constexpr int VPR = D / 8;
  constexpr int LPT = BN * VPR / NT;
  static_assert(BN * VPR % NT == 0, "tile must divide over the block");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T *sK = reinterpret_cast<T *>(smem_raw);  // [2][BN*KS]
  T *sV = sK + 2 * BN * KS;                 // [2][BN*VS]

  const int b = blockIdx.z, h = blockIdx.y;
  const int mt = gridDim.x - 1 - blockIdx.x;
  const int q0 = p.cu_q[b], sq = p.cu_q[b + 1] - q0;
  const int k0 = p.cu_k[b], sk = p.cu_k[b + 1] - k0;
  const int m0 = mt * BM;
  if (m0 >= sq) return;
  const int hkv = h / (p.hq / p.hk);
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int c = lane & 31, hh = lane >> 5;
  const int wrow0 = m0 + w * 32;
  const int row_q = wrow0 + c;
  const bool row_ok = row_q < sq;
  const int row_ld = row_ok ? row_q : sq - 1;

  Frag Qf[D / 16], dOf[D / 16];
  {
    const T *qp = reinterpret_cast<const T *>(p.q) + (int64_t)(q0 + row_ld) * p.q_stride + (int64_t)h * D;
    const T *dp = reinterpret_cast<const T *>(p.dout) + (int64_t)(q0 + row_ld) * p.do_stride + (int64_t)h * D;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      Qf[ks] = frag_ld<T>(qp + ks * 16 + 8 * hh);
      dOf[ks] = frag_ld<T>(dp + ks * 16 + 8 * hh);
    }
  }
  const float lse_c = row_ok ? p.lse[((int64_t)b * p.hq + h) * p.max_sq + row_q] * 1.4426950408889634f : INFINITY;
  const float del_c = row_ok ? p.delta[((int64_t)b * p.hq + h) * p.max_sq + row_q] : 0.f;

  const T *kg = reinterpret_cast<const T *>(p.k) + (int64_t)k0 * p.k_stride + (int64_t)hkv * D;
  const T *vg = reinterpret_cast<const T *>(p.v) + (int64_t)k0 * p.v_stride + (int64_t)hkv * D;
  int nk_end = sk;
  if (p.causal && m0 + BM < nk_end) nk_end = m0 + BM;
  const int ntiles = (nk_end + BN - 1) / BN;

  floatx16 dQt[D / 32];
#pragma unroll
  for (int t = 0; t < D / 32; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) dQt[t][v] = 0.f;

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
    const bool skip = p.causal && n0 > wrow0 + 31;
    if (!skip) {
      const T *tK = sK + st * BN * KS;
      const T *tV = sV + st * BN * VS;
      floatx16 S, dP;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        S[v] = 0.f;
        dP[v] = 0.f;
      }
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        const Frag ak = frag_ld<T>(tK + c * KS + ks * 16 + 8 * hh);
        S = M::mma(ak, Qf[ks], S);
        const Frag av = frag_ld<T>(tV + c * VS + ks * 16 + 8 * hh);
        dP = M::mma(av, dOf[ks], dP);
      }
      const bool need_mask = (p.causal && n0 + BN - 1 > wrow0) || (n0 + BN > sk);
      float dsv[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float pe = fast_exp2(S[v] * p.scale_log2 - lse_c);
        if (need_mask) {
          const int kv = n0 + acc_row(v, hh);
          if (kv >= sk || (p.causal && kv > row_q)) pe = 0.f;
        }
        dsv[v] = pe * (dP[v] - del_c);
      }
      Frag dSb[2];
      dSb[0] = frag_pack<T>(dsv);
      dSb[1] = frag_pack<T>(dsv + 8);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int t = 0; t < D / 32; ++t) {
          const Frag ak = frag_ld_tr<T>(tK, KS, 16 * s + 4 * hh, 16 * s + 8 + 4 * hh, 32 * t + 16 * ((lane >> 4) & 1), lane);
          dQt[t] = M::mma(ak, dSb[s], dQt[t]);
        }
      }
    }
    if (it + 1 < ntiles) sstore(st ^ 1);
    __syncthreads();
  }

  if (row_ok) {
    T *dqp = reinterpret_cast<T *>(p.dq) + (int64_t)(q0 + row_q) * p.dq_stride + (int64_t)h * D;
#pragma unroll
    for (int t = 0; t < D / 32; ++t)
#pragma unroll
      for (int vb = 0; vb < 4; ++vb) {
        struct alignas(8) { T v[4]; } a;
        if (p.dq_accumulate) {
          a = *reinterpret_cast<const decltype(a) *>(dqp + 32 * t + 8 * vb + 4 * hh);
#pragma unroll
          for (int e = 0; e < 4; ++e) a.v[e] = static_cast<T>(static_cast<float>(a.v[e]) + dQt[t][4 * vb + e] * p.scale);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) a.v[e] = static_cast<T>(dQt[t][4 * vb + e] * p.scale);
        }
        *reinterpret_cast<decltype(a) *>(dqp + 32 * t + 8 * vb + 4 * hh) = a;
      }
  }
}

// ---------------------------------------------------------------------------------------------
// Head dim 128, second-generation kernels: direct global->LDS copies into swizzled tiles
// (no staging registers, no bank conflicts), two pipeline stages held in separate LDS
// objects, causal work made uniform by pairing tile i with tile n-1-i.
// ---------------------------------------------------------------------------------------------

// dQ: 8 wavefronts = RG query row groups x SPLIT key splits (as the forward kernel); the
// partial dQ of the splits are added through LDS in split order.  As in the forward kernel
// the main loop is one rolled body whose global->LDS copies and LDS reads are written in
// assembly (scalar copy bases, XOR-derived fragment addresses, no compiler waits between
// copies in flight and reads); the copies are spread between the MFMAs.
template <typename T, int RG, int SPLIT, int BN>
__global__ void __launch_bounds__(512) attn_bwd_dq_d128_kernel(const AttnBwdParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  static_assert(BN == 32, "32-key tiles");
  constexpr int D = 128, BM = 32 * RG, NS = BN / 16;
  static_assert(RG * SPLIT == 8, "8 wavefronts per workgroup");
  constexpr int TILE = BN * D;
  constexpr int SLOT = SPLIT * TILE;              // elements of one K (or V) slot: the tiles of all splits
  constexpr int SLOTB = SLOT * (int)sizeof(T);
  constexpr int BPT = BN / 4;                     // 1 KB copy blocks per tile
  constexpr int CPW = SPLIT * 2 * BPT / 8;        // copy blocks per wavefront and iteration (4 or 8)
  static_assert(CPW == 4 || CPW == 8, "copy blocks per wavefront");
  __shared__ __attribute__((aligned(1024))) T sAll[4 * SLOT];   // K slots 0..1, V slots 0..1
  __shared__ float sDel[RG * 32];                               // delta of the workgroup's rows

  const int b = blockIdx.y;
  // the query heads of one kv head read the same K / V rows: keep a kv head on one XCD's L2
  const int ratio = p.hq / p.hk, P = gridDim.x / p.hq;
  int hkv, item;
  xcd_group_item(blockIdx.x, p.hk, ratio * P, hkv, item);
  const int h = hkv * ratio + item / P, px = item % P;
  const int q0 = p.cu_q[b], sq = p.cu_q[b + 1] - q0;
  const int k0 = p.cu_k[b], sk = p.cu_k[b + 1] - k0;
  const int nqt = (sq + BM - 1) / BM;
  const int causal = p.causal;
  const int k_stride = (int)p.k_stride, v_stride = (int)p.v_stride;
  const float scale_log2 = p.scale_log2;
  int qt[2], nq;
  if (causal) {
    const int pair = px;
    if (2 * pair >= nqt) return;
    qt[0] = nqt - 1 - pair; qt[1] = pair;
    nq = (qt[0] == qt[1]) ? 1 : 2;
  } else {
    if (px >= nqt) return;
    qt[0] = px; qt[1] = 0; nq = 1;
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: copy bookkeeping stays scalar
  const int c = lane & 31, hh = lane >> 5;
  const int rg = w % RG, sp = w / RG;
  const T *kg = reinterpret_cast<const T *>(p.k) + (int64_t)k0 * p.k_stride + (int64_t)hkv * D;
  const T *vg = reinterpret_cast<const T *>(p.v) + (int64_t)k0 * p.v_stride + (int64_t)hkv * D;
  const uint32_t ldsK = (uint32_t)(uintptr_t)sAll, ldsV = ldsK + 2 * SLOTB;

  // ---- copies: the CPW blocks of a wavefront are consecutive rows of ONE tile (K or V) -------------
  CopyLane cl0;
  cl0.l16 = lane & 15;
  cl0.lrow = lane >> 4;
  const int cp_tile = (w * CPW) / (2 * BPT);
  const int cp_v = ((w * CPW) % (2 * BPT)) / BPT;
  const int cp_r0 = 4 * ((w * CPW) % BPT);
  const int cp_stride = cp_v ? v_stride : k_stride;
  const T *cp_gt = cp_v ? vg : kg;
  const char *cp_g = reinterpret_cast<const char *>(cp_gt);
  const int cp_dst0 = cp_tile * TILE + cp_r0 * D;
  const uint32_t cp_step = (uint32_t)(4 * cp_stride) * (uint32_t)sizeof(T);
  uint32_t cp_off[4];                                 // both tiles use swz(row): chunk ^= 4 * (row % 4) + (row / 4) % 4
  {
    const uint32_t rowb = (uint32_t)(cl0.lrow * cp_stride) * (uint32_t)sizeof(T);
    const uint32_t chunk = (uint32_t)(cl0.l16 ^ (4 * cl0.lrow)) << 4;
#pragma unroll
    for (int x = 0; x < 4; ++x) cp_off[x] = rowb + (chunk ^ (uint32_t)(x << 4));
  }
  // ---- fragment reads: lane byte offsets inside a slot; other fragments by XOR / immediate offset ----
  const int r = lane & 15;
  const uint32_t rf_lane = (uint32_t)(sp * TILE * (int)sizeof(T) + c * 256 + ((hh ^ swz(c)) << 4));   // row c, chunk hh
  const int ta_x = 4 * (r >> 2) + hh;                 // transpose read of K: swz of rows 4*hh + r/4 (+8)
  const int t_lc = 2 * ((lane >> 4) & 1) + ((r & 3) >> 1);
  const uint32_t t_row = (uint32_t)(sp * TILE * (int)sizeof(T) + (4 * hh + (r >> 2)) * 256 + ((r & 3) & 1) * 8);
  const uint32_t ta_lane = t_row + (uint32_t)((t_lc ^ ta_x) << 4);
  const uint32_t tb_lane = t_row + 8 * 256 + (uint32_t)((t_lc ^ (ta_x + 2)) << 4);

  for (int qi = 0; qi < nq; ++qi) {
    const int m0 = qt[qi] * BM;
    const int wrow0 = m0 + rg * 32;
    const int row_q = wrow0 + c;
    const bool row_ok = row_q < sq;
    const int row_ld = row_ok ? row_q : sq - 1;
    Frag Qf[D / 16], dOf[D / 16];
    {
      const T *qp = reinterpret_cast<const T *>(p.q) + (int64_t)(q0 + row_ld) * p.q_stride + (int64_t)h * D;
      const T *dp = reinterpret_cast<const T *>(p.dout) + (int64_t)(q0 + row_ld) * p.do_stride + (int64_t)h * D;
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        Qf[ks] = frag_ld<T>(qp + ks * 16 + 8 * hh);
        dOf[ks] = frag_ld<T>(dp + ks * 16 + 8 * hh);
      }
    }
    const float lse_c = row_ok ? p.lse[((int64_t)b * p.hq + h) * p.max_sq + row_q] * 1.4426950408889634f : INFINITY;
    // delta = rowsum(dO * O) of this lane's row, formed by the first key split of each row group: the lane holds
    // one half of the row's dO (its k-step chunks), reads the same chunks of O, and the two halves meet through
    // the partner lane.  The other splits get it through LDS after the barrier that publishes the first tiles.
    // Split 0 also writes it out, together with the copy the dK/dV kernel streams (lse in exp2 units next to
    // delta, zeros in the rows that pad the last 32-row tile), so that no separate pass over dO and O is
    // needed.  The dK/dV kernel therefore runs after this one.
    float del_c = 0.f;
    if (sp == 0) {
      const T *op = reinterpret_cast<const T *>(p.out) + (int64_t)(q0 + row_ld) * p.o_stride + (int64_t)h * D;
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        const Frag of = frag_ld<T>(op + ks * 16 + 8 * hh);
#pragma unroll
        for (int j = 0; j < 8; ++j) del_c += to_f(dOf[ks][j]) * to_f(of[j]);
      }
      del_c += __shfl_xor(del_c, 32, 64);
      if (!row_ok) del_c = 0.f;
      if (hh == 0) {
        sDel[rg * 32 + c] = del_c;
        if (row_ok) p.delta[((int64_t)b * p.hq + h) * p.max_sq + row_q] = del_c;
        if (row_q < p.ld2_pitch) {
          const int64_t a2 = ((int64_t)b * p.hq + h) * p.ld2_pitch + row_q;
          p.ld2[a2] = row_ok ? lse_c : 0.f;
          p.ld2[p.ld2_plane + a2] = del_c;
        }
      }
    }
    int nk_end = sk;
    if (causal && m0 + BM < nk_end) nk_end = m0 + BM;
    const int ntiles = (nk_end + BN - 1) / BN;
    const int niter = (ntiles + SPLIT - 1) / SPLIT;
    const int n_fast = sk / (SPLIT * BN);          // iterations whose tiles lie wholly inside the keys

    floatx16 dQt[D / 32];
#pragma unroll
    for (int t = 0; t < D / 32; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) dQt[t][v] = 0.f;

    if (niter > 0 && cp_tile < ntiles)
      dma_tile32_general<T, CPW>(sAll + (cp_v ? 2 * SLOT : 0) + cp_dst0, cp_gt, cp_stride, 1, cp_tile * BN + cp_r0, cp_r0, sk, cl0);
    dma_wait_all();
    __syncthreads();
    del_c = sDel[rg * 32 + c];

    const char *cp_src = nullptr;
    uint32_t cp_dst = 0;
    bool fcopy = false;
#define DH_DQ_COPY(i)                                                                                   \
    do {                                                                                                \
      if ((i) < CPW && fcopy) {                                                                         \
        __builtin_amdgcn_sched_barrier(0);                                                              \
        dma_block_fast(cp_src, cp_off[(i) & 3], cp_dst);                                                \
        cp_src += cp_step;                                                                              \
        cp_dst += 1024;                                                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                              \
      }                                                                                                 \
    } while (0)

#pragma unroll 1
    for (int it = 0; it < niter; ++it) {
      const int nit = it + 1;
      const uint32_t cur = (uint32_t)((it & 1) * SLOTB), nxt = (uint32_t)((nit & 1) * SLOTB);
      const bool copy = nit < niter && nit * SPLIT + cp_tile < ntiles;
      fcopy = copy && nit < n_fast;
      cp_src = cp_g + (int64_t)((nit * SPLIT + cp_tile) * BN + cp_r0) * cp_stride * (int)sizeof(T);
      cp_dst = (cp_v ? ldsV : ldsK) + nxt + (uint32_t)(cp_dst0 * (int)sizeof(T));
      if (copy && !fcopy)
        dma_tile32_general<T, CPW>(sAll + (cp_v ? 2 * SLOT : 0) + (nit & 1) * SLOT + cp_dst0, cp_gt, cp_stride, 1,
                                   (nit * SPLIT + cp_tile) * BN + cp_r0, cp_r0, sk, cl0);
      const int tile_g = it * SPLIT + sp;
      const int n0 = tile_g * BN;
      const bool act = tile_g < ntiles && !(causal && n0 > wrow0 + 31);
      if (act) {
        uint32_t kb = ldsK + cur + rf_lane, vb = ldsV + cur + rf_lane;
        uint32_t ta = ldsK + cur + ta_lane, tb = ldsK + cur + tb_lane;
        asm volatile("" : "+v"(kb), "+v"(vb), "+v"(ta), "+v"(tb));   // derive the other addresses here, not ahead of the loop
        floatx16 S, dP;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          S[v] = 0.f;
          dP[v] = 0.f;
        }
        {
          // K and V row fragments are fetched one step ahead of the MFMAs that consume them.
          int4v fk[2], fv[2];
          lds_read128<0>(fk[0], kb);
          lds_read128<0>(fv[0], vb);
#pragma unroll
          for (int ks = 0; ks < D / 16; ++ks) {
            const int a = ks & 1, nx = (ks + 1) & 1;
            if (ks + 1 < D / 16) {
              lds_read128<0>(fk[nx], kb ^ (uint32_t)((ks + 1) << 5));
              lds_read128<0>(fv[nx], vb ^ (uint32_t)((ks + 1) << 5));
              lds_wait<2>(fk[a], fv[a]);
            } else {
              lds_wait<0>(fk[a], fv[a]);
            }
            S = M::mma(__builtin_bit_cast(Frag, fk[a]), Qf[ks], S);
            dP = M::mma(__builtin_bit_cast(Frag, fv[a]), dOf[ks], dP);
            if (CPW == 8) DH_DQ_COPY(ks);                            // all copy blocks go out in this phase, so
            if (CPW == 4 && (ks & 1)) DH_DQ_COPY(ks >> 1);           // that they have the rest of the iteration to land
          }
        }
        // dQ^T += K^T dS^T needs K^T fragments (transpose reads of the K tile): those of the first 16-key
        // step are requested now and land during the softmax part, those of the next step while the
        // current one multiplies.
        uint32_t ad[8];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          ad[2 * t] = ta ^ (uint32_t)(t << 6);
          ad[2 * t + 1] = tb ^ (uint32_t)(t << 6);
        }
        short4v f[2][8];
        lds_read_tr8<0>(f[0], ad);
        if ((causal && n0 + BN - 1 > wrow0) || (n0 + BN > sk)) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int kv = n0 + acc_row(v, hh);
            if (kv >= sk || (causal && kv > row_q)) S[v] = -INFINITY;     // P = dS = 0
          }
        }
        Frag dSb[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) {
          float dsv[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int v = 8 * s + j;
            const float pe = fast_exp2(S[v] * scale_log2 - lse_c);
            dsv[j] = pe * (dP[v] - del_c);
          }
          dSb[s] = frag_pack<T>(dsv);
        }
#pragma unroll
        for (int s = 0; s < NS; ++s) {
          short4v(&g)[8] = f[s & 1];
          if (s + 1 < NS) {
            lds_read_tr8<16 * 256>(f[(s + 1) & 1], ad);
            lds_wait<12>(g[0], g[1], g[2], g[3]);
          } else {
            lds_wait<4>(g[0], g[1], g[2], g[3]);
          }
          dQt[0] = M::mma(frag_join<T>(g[0], g[1]), dSb[s], dQt[0]);
          dQt[1] = M::mma(frag_join<T>(g[2], g[3]), dSb[s], dQt[1]);
          if (s + 1 < NS) lds_wait<8>(g[4], g[5], g[6], g[7]);
          else lds_wait<0>(g[4], g[5], g[6], g[7]);
          dQt[2] = M::mma(frag_join<T>(g[4], g[5]), dSb[s], dQt[2]);
          dQt[3] = M::mma(frag_join<T>(g[6], g[7]), dSb[s], dQt[3]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < CPW; ++i) DH_DQ_COPY(i);
      }
      dma_wait_all();
      __syncthreads();   // the next slots have landed, and everyone is done with the current ones
    }
#undef DH_DQ_COPY

    // add the splits' partial dQ through LDS, in split order: slot x = (s-1)*RG + g, 16 KB each
    float *xo = reinterpret_cast<float *>(sAll);
    static_assert((SPLIT - 1) * RG <= 6, "exchange slots");
    static_assert(4 * SLOT * sizeof(T) >= (size_t)(SPLIT - 1) * RG * 4096 * sizeof(float), "exchange area");
    if (sp > 0) {
      float *dst = xo + ((sp - 1) * RG + rg) * 4096;
#pragma unroll
      for (int t = 0; t < D / 32; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[(t * 16 + v) * 64 + lane] = dQt[t][v];
    }
    __syncthreads();
    if (sp == 0) {
#pragma unroll
      for (int s2 = 1; s2 < SPLIT; ++s2) {
        const float *src = xo + ((s2 - 1) * RG + rg) * 4096;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) dQt[t][v] += src[(t * 16 + v) * 64 + lane];
      }
      if (row_ok) {
        T *dqp = reinterpret_cast<T *>(p.dq) + (int64_t)(q0 + row_q) * p.dq_stride + (int64_t)h * D;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int vb = 0; vb < 4; ++vb) {
            struct alignas(8) { T v[4]; } a;
            if (p.dq_accumulate) {
              a = *reinterpret_cast<const decltype(a) *>(dqp + 32 * t + 8 * vb + 4 * hh);
#pragma unroll
              for (int e = 0; e < 4; ++e) a.v[e] = static_cast<T>(static_cast<float>(a.v[e]) + dQt[t][4 * vb + e] * p.scale);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) a.v[e] = static_cast<T>(dQt[t][4 * vb + e] * p.scale);
            }
            *reinterpret_cast<decltype(a) *>(dqp + 32 * t + 8 * vb + 4 * hh) = a;
          }
      }
    }
    __syncthreads();
  }
}

// dQ from the dS blocks that the dK/dV kernel left in the workspace: dQ^T[d, q] += K^T[d, key] dS^T[key, q], one
// matrix product instead of the three of the recomputing kernel above (which stays for shapes whose dS would not
// fit the workspace).  Same workgroup shape: 2 query row groups x 4 key splits, 32-key steps, the splits' partial
// sums added through LDS in split order.  A step needs the K tile of its split (8 KB, swizzled rows, transpose
// reads as above) and one 2 KB dS block per row group, copied as it lies in memory; its transpose reads pick,
// for a 16-lane group of query columns, the 8-byte pieces (u, hh) of four consecutive keys, which puts query
// row n of the tile on lane n.  The kernel streams 2 bytes of dS per 256 flops: it is bound by memory.
template <typename T>
__global__ void __launch_bounds__(512) attn_bwd_dq2_d128_kernel(const AttnBwdParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int D = 128, RG = 2, SPLIT = 4, BN = 32, BM = 32 * RG;
  constexpr int TILE = BN * D;                         // elements of one K tile
  constexpr int TILEB = TILE * (int)sizeof(T);
  constexpr int SLOTB = SPLIT * TILEB;                 // the K tiles of all splits: one stage
  constexpr int DSB = RG * 2048;                       // the dS blocks of one split (one per row group)
  constexpr int DSLOTB = SPLIT * DSB;
  constexpr int NST = 3;                               // stages: the copies of a step go out two steps ahead of it
  __shared__ __attribute__((aligned(1024))) char sAll[NST * SLOTB + NST * DSLOTB];   // 144 KB

  const int b = blockIdx.y;
  // a head's dS blocks were written from one XCD (the dK/dV kernel keeps a head group there): read them from the
  // same one; the K rows of the kv head are small next to them
  const int ratio = p.hq / p.hk, P = gridDim.x / p.hq;
  int h, px;
  xcd_group_item(blockIdx.x, p.hq, P, h, px);
  const int hkv = h / ratio;
  const int q0 = p.cu_q[b], sq = p.cu_q[b + 1] - q0;
  const int k0 = p.cu_k[b], sk = p.cu_k[b + 1] - k0;
  const int nqt = (sq + BM - 1) / BM;
  const int causal = p.causal;
  const int k_stride = (int)p.k_stride;
  int qt[2], nq;
  if (causal) {
    if (2 * px >= nqt) return;
    qt[0] = nqt - 1 - px; qt[1] = px;
    nq = (qt[0] == qt[1]) ? 1 : 2;
  } else {
    if (px >= nqt) return;
    qt[0] = px; qt[1] = 0; nq = 1;
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hh = lane >> 5;
  const int rg = w % RG, sp = w / RG;
  const T *kg = reinterpret_cast<const T *>(p.k) + (int64_t)k0 * p.k_stride + (int64_t)hkv * D;
  const char *kg_b = reinterpret_cast<const char *>(kg);
  const uint32_t ldsK = (uint32_t)(uintptr_t)sAll, ldsD = ldsK + NST * SLOTB;

  // ---- copies of wavefront w: rows [16 half, 16 half + 16) of the K tile of split w / 2 (four 1 KB blocks) and the
  // dS block of row group `half` of that split (two 1 KB blocks) -------------------------------------------------
  CopyLane cl0;
  cl0.l16 = lane & 15;
  cl0.lrow = lane >> 4;
  const int csp = w >> 1, half = w & 1;
  const uint32_t cp_step = (uint32_t)(4 * k_stride) * (uint32_t)sizeof(T);
  uint32_t cp_off[4];
  {
    const uint32_t rowb = (uint32_t)(cl0.lrow * k_stride) * (uint32_t)sizeof(T);
    const uint32_t chunk = (uint32_t)(cl0.l16 ^ (4 * cl0.lrow)) << 4;
#pragma unroll
    for (int x = 0; x < 4; ++x) cp_off[x] = rowb + (chunk ^ (uint32_t)(x << 4));
  }
  // The dK/dV kernel wrote a dS block as two fragments of 64 lanes x 16 bytes (piece 64 s + L is lane L of fragment
  // s).  The transpose reads below fetch, per instruction, the pieces L = 32 b + 8 t + 4 hh + j of both fragments
  // (t fixed; j = 0..3, b = 0..1): copied as they lie, the four 64-byte runs (s, b) of a half wavefront fall on the
  // same 16 banks.  So the copy permutes: LDS position 64 hh + 16 t + 8 s + 4 b + j holds that piece (lane l of the
  // copy for half hh fetches the piece with j = l % 4, b = l / 4 % 2, s = l / 8 % 2, t = l / 16), and the 16 pieces of
  // a half wavefront's read are 256 consecutive bytes.
  const uint32_t ds_lane = 16u * (uint32_t)(64 * ((lane >> 3) & 1) + 32 * ((lane >> 2) & 1) + 8 * ((lane >> 4) & 3) + (lane & 3));
  const int64_t ds_head = ((int64_t)b * p.hq + h) * p.ds_nqt;
  const char *ds_b = reinterpret_cast<const char *>(p.ds);

  // ---- fragment reads ------------------------------------------------------------------------------------------
  const int r = lane & 15;
  const int ta_x = 4 * (r >> 2) + hh;                 // transpose reads of K: swz of rows 4*hh + r/4 (+8)
  const int t_lc = 2 * ((lane >> 4) & 1) + ((r & 3) >> 1);
  const uint32_t t_row = (uint32_t)(sp * TILEB + (4 * hh + (r >> 2)) * 256 + ((r & 3) & 1) * 8);
  const uint32_t ta_lane = t_row + (uint32_t)((t_lc ^ ta_x) << 4);
  const uint32_t tb_lane = t_row + 8 * 256 + (uint32_t)((t_lc ^ (ta_x + 2)) << 4);
  // dS block: piece (s = 16-lane group, hh_p = r % 2) of key 4 hh + r / 4, half u = (r % 4) / 2 of the piece
  const uint32_t db_lane = (uint32_t)(sp * DSB + rg * 2048 + ((64 * hh + 8 * ((lane >> 4) & 1) + 4 * (r & 1) + (r >> 2)) * 16) +
                                      ((r & 3) >> 1) * 8);        // + 256 t

  for (int qi = 0; qi < nq; ++qi) {
    const int m0 = qt[qi] * BM;
    const int wrow0 = m0 + rg * 32;
    const int row_q = wrow0 + c;
    const bool row_ok = row_q < sq;
    int nk_end = sk;
    if (causal && m0 + BM < nk_end) nk_end = m0 + BM;
    const int ntiles = (nk_end + BN - 1) / BN;
    const int niter = (ntiles + SPLIT - 1) / SPLIT;
    const int n_fast = sk / (SPLIT * BN);          // iterations whose K tiles lie wholly inside the keys
    const int64_t ds_row = (ds_head + (m0 >> 5) + half) * p.ds_nkb;   // the copied block row: query tile of row group `half`

    floatx16 dQt[D / 32];
#pragma unroll
    for (int t = 0; t < D / 32; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) dQt[t][v] = 0.f;

    auto issue = [&](int it) {
      const int tile = it * SPLIT + csp;
      if (tile >= ntiles) return;
      const uint32_t stK = (uint32_t)((it % NST) * SLOTB), stD = (uint32_t)((it % NST) * DSLOTB);
      if (it < n_fast) {
        const char *src = kg_b + (int64_t)(tile * BN + 16 * half) * k_stride * (int)sizeof(T);
        uint32_t dst = ldsK + stK + (uint32_t)(csp * TILEB + 16 * half * 256);
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          dma_block_fast(src, cp_off[x], dst);
          src += cp_step;
          dst += 1024;
        }
      } else {
        dma_tile32_general<T, 4>(reinterpret_cast<T *>(sAll + stK + csp * TILEB) + 16 * half * D, kg, k_stride, 1,
                                 tile * BN + 16 * half, 16 * half, sk, cl0);
      }
      const char *dsrc = ds_b + (ds_row + tile) * 2048;
      const uint32_t ddst = ldsD + stD + (uint32_t)(csp * DSB + half * 2048);
      dma_block_fast(dsrc, ds_lane, ddst);
      dma_block_fast(dsrc + 64, ds_lane, ddst + 1024);
    };

    // Steps 0 and 1 go out now; in the loop, step it + 2 goes out at the top of step it and the wait at the bottom
    // leaves the newest step's copies in flight (6 per wavefront, or none: vmcnt counts in issue order).
    if (niter > 0) issue(0);
    if (niter > 1) issue(1);
    if (niter > 1 && 1 * SPLIT + csp < ntiles && 1 < n_fast) {
      asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    } else {
      dma_wait_all();
      __syncthreads();
    }

#pragma unroll 1
    for (int it = 0; it < niter; ++it) {
      if (it + 2 < niter) issue(it + 2);              // has two steps to land
      const int tile_g = it * SPLIT + sp;
      const int n0 = tile_g * BN;
      const bool act = tile_g < ntiles && !(causal && n0 > wrow0 + 31);
      if (act) {
        const uint32_t curK = ldsK + (uint32_t)((it % NST) * SLOTB), curD = ldsD + (uint32_t)((it % NST) * DSLOTB);
        uint32_t ta = curK + ta_lane, tb = curK + tb_lane, db = curD + db_lane;
        asm volatile("" : "+v"(ta), "+v"(tb), "+v"(db));
        // LDS reads in assembly (the compiler would hold them behind every copy in flight): the four dS pieces,
        // the K^T fragments of the first 16 keys, then those of the second while the first multiply
        uint32_t ad[8];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          ad[2 * t] = ta ^ (uint32_t)(t << 6);
          ad[2 * t + 1] = tb ^ (uint32_t)(t << 6);
        }
        short4v bq[4], f0[8], f1[8];
        lds_read_tr4<256>(bq, db);
        lds_read_tr8<0>(f0, ad);
        lds_wait<4>(bq[0], bq[1], bq[2], bq[3]);
        lds_wait<4>(f0[0], f0[1], f0[2], f0[3]);
        lds_read_tr8<16 * 256>(f1, ad);
        const Frag dS0 = frag_join<T>(bq[0], bq[1]), dS1 = frag_join<T>(bq[2], bq[3]);
        dQt[0] = M::mma(frag_join<T>(f0[0], f0[1]), dS0, dQt[0]);
        dQt[1] = M::mma(frag_join<T>(f0[2], f0[3]), dS0, dQt[1]);
        lds_wait<8>(f0[4], f0[5], f0[6], f0[7]);
        dQt[2] = M::mma(frag_join<T>(f0[4], f0[5]), dS0, dQt[2]);
        dQt[3] = M::mma(frag_join<T>(f0[6], f0[7]), dS0, dQt[3]);
        lds_wait<4>(f1[0], f1[1], f1[2], f1[3]);
        dQt[0] = M::mma(frag_join<T>(f1[0], f1[1]), dS1, dQt[0]);
        dQt[1] = M::mma(frag_join<T>(f1[2], f1[3]), dS1, dQt[1]);
        lds_wait<0>(f1[4], f1[5], f1[6], f1[7]);
        dQt[2] = M::mma(frag_join<T>(f1[4], f1[5]), dS1, dQt[2]);
        dQt[3] = M::mma(frag_join<T>(f1[6], f1[7]), dS1, dQt[3]);
      }
      // step it + 1 must have landed; the copies of step it + 2 (the newest 6 of this wavefront, if it issued them
      // in the fast form) may stay in flight
      // (__syncthreads() would drain them: it waits for every memory operation before its barrier)
      if (it + 2 < niter && (it + 2) * SPLIT + csp < ntiles && it + 2 < n_fast) {
        asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      } else {
        dma_wait_all();
        __syncthreads();
      }
    }

    // add the splits' partial dQ through LDS, in split order: slot x = (s-1)*RG + g, 16 KB each
    float *xo = reinterpret_cast<float *>(sAll);
    static_assert(sizeof(sAll) >= (size_t)(SPLIT - 1) * RG * 4096 * sizeof(float), "exchange area");
    if (sp > 0) {
      float *dst = xo + ((sp - 1) * RG + rg) * 4096;
#pragma unroll
      for (int t = 0; t < D / 32; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[(t * 16 + v) * 64 + lane] = dQt[t][v];
    }
    __syncthreads();
    if (sp == 0) {
#pragma unroll
      for (int s2 = 1; s2 < SPLIT; ++s2) {
        const float *src = xo + ((s2 - 1) * RG + rg) * 4096;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) dQt[t][v] += src[(t * 16 + v) * 64 + lane];
      }
      if (row_ok) {
        T *dqp = reinterpret_cast<T *>(p.dq) + (int64_t)(q0 + row_q) * p.dq_stride + (int64_t)h * D;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int vb = 0; vb < 4; ++vb) {
            struct alignas(8) { T v[4]; } a;
            if (p.dq_accumulate) {
              a = *reinterpret_cast<const decltype(a) *>(dqp + 32 * t + 8 * vb + 4 * hh);
#pragma unroll
              for (int e = 0; e < 4; ++e) a.v[e] = static_cast<T>(static_cast<float>(a.v[e]) + dQt[t][4 * vb + e] * p.scale);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) a.v[e] = static_cast<T>(dQt[t][4 * vb + e] * p.scale);
            }
            *reinterpret_cast<decltype(a) *>(dqp + 32 * t + 8 * vb + 4 * hh) = a;
          }
      }
    }
    __syncthreads();
  }
}

template <typename T>
static int launch_dq2_d128(const AttnBwdParams &p, int batch, hipStream_t st) {
  constexpr int BM = 64;
  const int nqt = (int)cdiv(p.max_sq, BM);
  dim3 grid((unsigned)((p.causal ? (nqt + 1) / 2 : nqt) * p.hq), (unsigned)batch);
  hipLaunchKernelGGL((attn_bwd_dq2_d128_kernel<T>), grid, dim3(512), 0, st, p);
  return DH_OK;
}

template <typename T, int RG, int SPLIT, int BN>
static int launch_dq_d128(const AttnBwdParams &p, int batch, hipStream_t st) {
  constexpr int BM = 32 * RG;
  const int nqt = (int)cdiv(p.max_sq, BM);
  dim3 grid((unsigned)((p.causal ? (nqt + 1) / 2 : nqt) * p.hq), (unsigned)batch);
  hipLaunchKernelGGL((attn_bwd_dq_d128_kernel<T, RG, SPLIT, BN>), grid, dim3(512), 0, st, p);
  return DH_OK;
}

// dK/dV with eight wavefronts: 2 key row groups (32 rows each) x 4 query splits, i.e. two wavefronts per
// SIMD whose matrix and softmax phases interleave.  To fit that into 256 registers per wavefront the K / V
// tiles of the workgroup live in LDS (read as row fragments every iteration) instead of registers, the
// accumulators are ordinary variables, and lse / delta of a query tile come straight from memory (one
// aligned 128-byte run per tile and plane), loaded one iteration ahead.  LDS: two stages of four Q + dO tile
// pairs (128 KB) + the K and V tiles (32 KB).  The splits' partial dK/dV are added through LDS in a fixed
// order.  Causal: the workgroup owns key tiles j and n-1-j, so every workgroup does the same amount of
// work.  The main loop is one rolled body; the Q / dO tiles of the next iteration come in with assembly
// copies (scalar bases) issued between the matrix instructions.
template <typename T, bool STORE_DS>
__global__ void __launch_bounds__(512) attn_bwd_dkv_d128_kernel(const AttnBwdParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int D = 128, KG = 2, QSPLIT = 4, BN = 32 * KG, BM = 32;
  constexpr int QT = BM * D;                          // elements of one Q (or dO) tile
  constexpr int QTB = QT * (int)sizeof(T);
  constexpr int SLOT = 2 * QT;                        // Q tile, dO tile
  constexpr int SLOTB = SLOT * (int)sizeof(T);
  constexpr int STAGE = QSPLIT * SLOT;
  constexpr int STAGEB = STAGE * (int)sizeof(T);
  constexpr int KVT = BN * D;                         // elements of the K (or V) tile
  constexpr int KVTB = KVT * (int)sizeof(T);
  __shared__ __attribute__((aligned(1024))) T sAll[2 * STAGE + 2 * KVT];

  const int b = blockIdx.y;
  const int G = p.hk * p.hsplit;
  int hg, px;
  xcd_group_item(blockIdx.x, G, gridDim.x / G, hg, px);
  const int hkv = hg / p.hsplit, hs = hg % p.hsplit;
  const int q0 = p.cu_q[b], sq = p.cu_q[b + 1] - q0;
  const int k0 = p.cu_k[b], sk = p.cu_k[b + 1] - k0;
  const int nkt = (sk + BN - 1) / BN;
  const int causal = p.causal;
  const int q_stride = (int)p.q_stride, do_stride = (int)p.do_stride;
  const float scale_log2 = p.scale_log2;
  int kt[2], nk;
  if (causal) {
    const int pair = px;
    if (2 * pair >= nkt) return;
    kt[0] = pair; kt[1] = nkt - 1 - pair;             // heavy (early keys) first
    nk = (kt[0] == kt[1]) ? 1 : 2;
  } else {
    if (px >= nkt) return;
    kt[0] = px; kt[1] = 0; nk = 1;
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: copy bookkeeping stays scalar
  const int c = lane & 31, hh = lane >> 5;
  const int kg = w % KG, qs = w / KG;
  const int ratio = p.hq / p.hk;
  const int hper = ratio / p.hsplit;
  const int h_first = hkv * ratio + hs * hper;
  const uint32_t lds0 = (uint32_t)(uintptr_t)sAll;
  const uint32_t ldsKV = lds0 + 2u * STAGEB;

  // ---- copies: wavefront w brings one whole tile per iteration: Q (w even) or dO (w odd) of split w / 2 ----
  CopyLane cl0;
  cl0.l16 = lane & 15;
  cl0.lrow = lane >> 4;
  const int cp_slot = w >> 1, cp_do = w & 1;
  const int cp_stride = cp_do ? do_stride : q_stride;
  const T *cp_gt = reinterpret_cast<const T *>(cp_do ? p.dout : p.q) + (int64_t)q0 * cp_stride;
  const char *cp_g = reinterpret_cast<const char *>(cp_gt);
  const int cp_dst0 = cp_slot * SLOT + cp_do * QT;    // elements inside a stage
  const uint32_t cp_step = (uint32_t)(4 * cp_stride) * (uint32_t)sizeof(T);
  uint32_t cp_off[4];                                 // tiles use swz(row): chunk ^= 4 * (row % 4) + (row / 4) % 4
  {
    const uint32_t rowb = (uint32_t)(cl0.lrow * cp_stride) * (uint32_t)sizeof(T);
    const uint32_t chunk = (uint32_t)(cl0.l16 ^ (4 * cl0.lrow)) << 4;
#pragma unroll
    for (int x = 0; x < 4; ++x) cp_off[x] = rowb + (chunk ^ (uint32_t)(x << 4));
  }
  typedef __attribute__((address_space(3))) const Frag *lds_frag;
  typedef short4v __attribute__((address_space(3))) *lds_tr;

  for (int ki = 0; ki < nk; ++ki) {
    const int j0 = kt[ki] * BN;
    const int jw0 = j0 + 32 * kg;
    const int jrow = jw0 + c;
    // this workgroup's K and V tiles -> LDS: wavefronts 0, 1 bring the two halves of K, wavefronts 2, 3 of V
    if (w < 4) {
      const int half = w & 1, isv = w >> 1;
      const T *gsrc = reinterpret_cast<const T *>(isv ? p.v : p.k) + (int64_t)k0 * (isv ? p.v_stride : p.k_stride) +
                      (int64_t)hkv * D;
      dma_tile32_general<T, 8>(sAll + 2 * STAGE + isv * KVT + half * 32 * D, gsrc, (int)(isv ? p.v_stride : p.k_stride), 1,
                               j0 + 32 * half, 0, sk, cl0);
    }
    floatx16 dKt[D / 32], dVt[D / 32];
#pragma unroll
    for (int t = 0; t < D / 32; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        dKt[t][v] = 0.f;
        dVt[t][v] = 0.f;
      }
    const int i_begin = causal ? (j0 / BM) * BM : 0;
    const int ntq = i_begin < sq ? (sq - i_begin + BM - 1) / BM : 0;
    const int it_per_head = (ntq + QSPLIT - 1) / QSPLIT;
    const int niter = it_per_head * hper;

    auto issue_general = [&](int st, int g, int ti) {
      const int h = h_first + g;
      const int tq = ti * QSPLIT + cp_slot;
      if (tq < ntq)
        dma_tile32_general<T, 8>(sAll + st + cp_dst0, cp_gt + (int64_t)h * D, cp_stride, 1, i_begin + tq * BM, 0, sq, cl0);
    };
    // lse (exp2 units) and delta of the rows 8*vb + 4*hh + e of this wavefront's query tile in iteration (g, ti)
    floatx4 l4[4], d4[4];
    auto load_ld = [&](int g, int ti) {
      const int tq = ti * QSPLIT + qs;
      if (tq < ntq) {
        int lx = lane;
        asm volatile("" : "+v"(lx));       // the address is formed here, not kept across the loop
        const float *src = p.ld2 + ((int64_t)b * p.hq + (h_first + g)) * p.ld2_pitch + (i_begin + tq * BM) + 4 * (lx >> 5);
#pragma unroll
        for (int vb = 0; vb < 4; ++vb) {
          l4[vb] = *reinterpret_cast<const floatx4 *>(src + 8 * vb);
          d4[vb] = *reinterpret_cast<const floatx4 *>(src + p.ld2_plane + 8 * vb);
        }
      }
    };
#pragma unroll
    for (int vb = 0; vb < 4; ++vb)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        l4[vb][e] = 0.f;
        d4[vb][e] = 0.f;
      }

    if (niter > 0) {
      issue_general(0, 0, 0);
      load_ld(0, 0);
    }
    dma_wait_all();
    __syncthreads();

    const char *cp_src = nullptr;
    uint32_t cp_dst = 0;
    bool fcopy = false;
#define DH_DKV_COPY(i)                                                                                  \
    do {                                                                                                \
      if (fcopy) {                                                                                      \
        __builtin_amdgcn_sched_barrier(0);                                                              \
        dma_block_fast(cp_src, cp_off[(i) & 3], cp_dst);                                                \
        cp_src += cp_step;                                                                              \
        cp_dst += 1024;                                                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                              \
      }                                                                                                 \
    } while (0)

    int g = 0, ti = 0;                                // head and step of iteration it
#pragma unroll 1
    for (int it = 0; it < niter; ++it) {
      int gn = g, tn = ti + 1;                        // ... and of iteration it + 1
      if (tn == it_per_head) { tn = 0; ++gn; }
      const bool have_next = it + 1 < niter;
      const uint32_t cur = lds0 + (uint32_t)((it & 1) * STAGEB);
      const int nxt_el = ((it + 1) & 1) * STAGE;
      {
        const int hn = h_first + gn;
        const int tq = tn * QSPLIT + cp_slot;
        const int row0 = i_begin + tq * BM;
        const bool copy = have_next && tq < ntq;
        fcopy = copy && row0 + BM <= sq;
        cp_src = cp_g + ((int64_t)row0 * cp_stride + (int64_t)hn * D) * (int)sizeof(T);
        cp_dst = lds0 + (uint32_t)((nxt_el + cp_dst0) * (int)sizeof(T));
        if (copy && !fcopy)
          dma_tile32_general<T, 8>(sAll + nxt_el + cp_dst0, cp_gt + (int64_t)hn * D, cp_stride, 1, row0, 0, sq, cl0);
      }
      const int tq = ti * QSPLIT + qs;
      const int i0 = i_begin + tq * BM;
      const bool act = tq < ntq && !(causal && i0 + BM - 1 < jw0);
      if (act) {
        // Fragment reads: lane byte offsets inside a slot; the other fragments are reached by XOR / immediate
        // offsets.  They are recomputed from the lane id here (a dozen instructions) rather than kept in
        // registers across the loop, which has none to spare.
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int lc = ln & 31, lh = ln >> 5, r = ln & 15;
        const uint32_t rowsw = (uint32_t)(lc * 256 + ((lh ^ swz(lc)) << 4));            // row lc, chunk lh
        const int ta_x = 4 * (r >> 2) + lh;                 // transpose reads: swz of rows 4*lh + r/4 (+8)
        const int t_lc = 2 * ((ln >> 4) & 1) + ((r & 3) >> 1);
        const uint32_t t_row = (uint32_t)((4 * lh + (r >> 2)) * 256 + ((r & 3) & 1) * 8);
        const uint32_t slot = cur + (uint32_t)(qs * SLOTB);
        uint32_t qb = slot + rowsw, kb = ldsKV + (uint32_t)(kg * 32 * 256) + rowsw;
        uint32_t ta = slot + t_row + (uint32_t)((t_lc ^ ta_x) << 4);
        uint32_t tb = slot + t_row + 8 * 256 + (uint32_t)((t_lc ^ (ta_x + 2)) << 4);
        asm volatile("" : "+v"(qb), "+v"(ta), "+v"(tb), "+v"(kb));   // derive the other addresses here
        floatx16 S, dP;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          S[v] = 0.f;
          dP[v] = 0.f;
        }
        // S = Q K^T and dP = dO V^T with the key index on lanes; the four fragments of step ks + 1 are
        // requested before the matrix instructions of step ks (the scheduling barriers pin that order)
        {
          Frag fq[2], fk[2], fo[2], fv[2];
          fq[0] = *(lds_frag)(qb);
          fk[0] = *(lds_frag)(kb);
          fo[0] = *(lds_frag)(qb + QTB);
          fv[0] = *(lds_frag)(kb + KVTB);
#pragma unroll
          for (int ks = 0; ks < D / 16; ++ks) {
            const int cb = ks & 1, nb = cb ^ 1;
            if (ks + 1 < D / 16) {
              const uint32_t aq = qb ^ (uint32_t)((ks + 1) << 5), ak = kb ^ (uint32_t)((ks + 1) << 5);
              fq[nb] = *(lds_frag)(aq);
              fk[nb] = *(lds_frag)(ak);
              fo[nb] = *(lds_frag)(aq + QTB);
              fv[nb] = *(lds_frag)(ak + KVTB);
            }
            __builtin_amdgcn_sched_barrier(0);
            S = M::mma(fq[cb], fk[cb], S);
            dP = M::mma(fo[cb], fv[cb], dP);
            __builtin_amdgcn_sched_barrier(0);
            DH_DKV_COPY(ks);                          // one copy block per step: all eight are out before the softmax
          }
        }
        if ((causal && i0 < jw0 + 31) || (i0 + BM > sq) || (STORE_DS && jw0 + 32 > sk)) {
          // masked scores become -inf, i.e. P = dS = 0 (lse and delta of rows past the sequence end are zeros);
          // keys past the end matter only when dS is kept: the dQ product would meet them
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int i = i0 + acc_row(v, hh);
            if (i >= sq || (causal && jrow > i) || (STORE_DS && jrow >= sk)) S[v] = -INFINITY;
          }
        }
        Frag Pb[2], dSb[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          float pv[8], dsv[8];
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const int vb = 2 * s + u;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int v = 4 * vb + e;
              const float pe = fast_exp2(S[v] * scale_log2 - l4[vb][e]);
              pv[4 * u + e] = pe;
              dsv[4 * u + e] = pe * (dP[v] - d4[vb][e]);
            }
          }
          Pb[s] = frag_pack<T>(pv);
          dSb[s] = frag_pack<T>(dsv);
        }
        if (STORE_DS) {
          // the packed dS fragments go out as they are, 1 KB per fragment and wavefront
          const int64_t blk = (((int64_t)b * p.hq + (h_first + g)) * p.ds_nqt + (i0 >> 5)) * p.ds_nkb + (jw0 >> 5);
          int lx = lane;
          asm volatile("" : "+v"(lx));
          Frag *dst = reinterpret_cast<Frag *>(reinterpret_cast<char *>(p.ds) + blk * 2048) + lx;
          dst[0] = dSb[0];
          dst[64] = dSb[1];
        }
        if (have_next) load_ld(gn, tn);               // next tile's lse / delta, in flight across the barrier
        // dV^T += dO^T P and dK^T += Q^T dS; the eight copy blocks of this wavefront go out in between.
        // Step u = (s, which, t): which = 0 reads dO^T (for dV), 1 reads Q^T (for dK); the fragments of
        // step u + 1 are requested before the matrix instruction of step u.
        {
          constexpr int AH = 2;                      // steps requested ahead
          short4v x0[AH + 1], x1[AH + 1];
          auto rd = [&](int u) {
            const int sx = u >> 3, which = (u >> 2) & 1, t = u & 3;
            const uint32_t a0 = (ta ^ (uint32_t)(t << 6)) + (uint32_t)(sx * 16 * 256) + (which ? 0u : (uint32_t)QTB);
            const uint32_t a1 = (tb ^ (uint32_t)(t << 6)) + (uint32_t)(sx * 16 * 256) + (which ? 0u : (uint32_t)QTB);
            x0[u % (AH + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(a0));
            x1[u % (AH + 1)] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(a1));
          };
#pragma unroll
          for (int u = 0; u < AH; ++u) rd(u);
#pragma unroll
          for (int u = 0; u < 16; ++u) {
            const int sx = u >> 3, which = (u >> 2) & 1, t = u & 3, cb = u % (AH + 1);
            if (u + AH < 16) rd(u + AH);
            __builtin_amdgcn_sched_barrier(0);
            if (which == 0) dVt[t] = M::mma(frag_join<T>(x0[cb], x1[cb]), Pb[sx], dVt[t]);
            else dKt[t] = M::mma(frag_join<T>(x0[cb], x1[cb]), dSb[sx], dKt[t]);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      } else {
        if (have_next) load_ld(gn, tn);
#pragma unroll
        for (int i = 0; i < 8; ++i) DH_DKV_COPY(i);
      }
      g = gn;
      ti = tn;
      dma_wait_all();
      __syncthreads();   // the next stage has landed, and everyone is done with the current one
    }
#undef DH_DKV_COPY

    // add the splits' partial sums through LDS in a fixed order: (0 += 2, 1 += 3), then 0 += 1.
    // Slot (split, key group) holds dK then dV, 16 KB each, in the stage area.
    static_assert(2 * STAGE * sizeof(T) >= (size_t)2 * KG * 2 * 4096 * sizeof(float), "exchange area");
    typedef __attribute__((address_space(3))) float *lds_f;
#pragma unroll
    for (int round = 0; round < 2; ++round) {
      const int senders_from = round == 0 ? 2 : 1, senders_to = round == 0 ? 4 : 2;
      if (qs >= senders_from && qs < senders_to) {
        int lx = lane;
        asm volatile("" : "+v"(lx));       // one base register + immediate offsets, computed here
        const uint32_t xb = lds0 + (uint32_t)((((qs - senders_from) * KG + kg) * 2 * 4096 + lx) * 4);
        lds_f dst = (lds_f)(xb);
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            dst[(t * 16 + v) * 64] = dKt[t][v];
            dst[4096 + (t * 16 + v) * 64] = dVt[t][v];
          }
      }
      __syncthreads();
      if (qs < senders_from) {
        int lx = lane;
        asm volatile("" : "+v"(lx));
        const uint32_t xb = lds0 + (uint32_t)(((qs * KG + kg) * 2 * 4096 + lx) * 4);
        lds_f src = (lds_f)(xb);
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            dKt[t][v] += src[(t * 16 + v) * 64];
            dVt[t][v] += src[4096 + (t * 16 + v) * 64];
          }
      }
      __syncthreads();
    }
    // the store addresses are derived from the lane id here, so that nothing but the id lives through the loop
    int ln = lane;
    asm volatile("" : "+v"(ln));
    if (qs == 0 && jw0 + (ln & 31) < sk) {
      const int hh = ln >> 5, jrow = jw0 + (ln & 31);
      if (p.hsplit == 1) {
        T *dkp = reinterpret_cast<T *>(p.dk) + (int64_t)(k0 + jrow) * p.dk_stride + (int64_t)hkv * D;
        T *dvp = reinterpret_cast<T *>(p.dv) + (int64_t)(k0 + jrow) * p.dv_stride + (int64_t)hkv * D;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int vb = 0; vb < 4; ++vb) {
            struct alignas(8) { T v[4]; } a, bq;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              a.v[e] = static_cast<T>(dKt[t][4 * vb + e] * p.scale);
              bq.v[e] = static_cast<T>(dVt[t][4 * vb + e]);
            }
            *reinterpret_cast<decltype(a) *>(dkp + 32 * t + 8 * vb + 4 * hh) = a;
            *reinterpret_cast<decltype(bq) *>(dvp + 32 * t + 8 * vb + 4 * hh) = bq;
          }
      } else {
        const int64_t off = (((int64_t)hs * p.total_k + (k0 + jrow)) * p.hk + hkv) * D;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int vb = 0; vb < 4; ++vb) {
            *reinterpret_cast<float4 *>(p.dk_part + off + 32 * t + 8 * vb + 4 * hh) =
                make_float4(dKt[t][4 * vb] * p.scale, dKt[t][4 * vb + 1] * p.scale, dKt[t][4 * vb + 2] * p.scale,
                            dKt[t][4 * vb + 3] * p.scale);
            *reinterpret_cast<float4 *>(p.dv_part + off + 32 * t + 8 * vb + 4 * hh) =
                make_float4(dVt[t][4 * vb], dVt[t][4 * vb + 1], dVt[t][4 * vb + 2], dVt[t][4 * vb + 3]);
          }
      }
    }
    __syncthreads();   // the K / V tiles and the exchange area are rewritten by the next key tile
  }
}

template <typename T>
static int launch_dkv_d128(const AttnBwdParams &p, int batch, int max_sk, hipStream_t st) {
  const int nkt = (int)cdiv(max_sk, 64);
  dim3 grid((unsigned)((p.causal ? (nkt + 1) / 2 : nkt) * p.hk * p.hsplit), (unsigned)batch);
  if (p.ds) hipLaunchKernelGGL((attn_bwd_dkv_d128_kernel<T, true>), grid, dim3(512), 0, st, p);
  else hipLaunchKernelGGL((attn_bwd_dkv_d128_kernel<T, false>), grid, dim3(512), 0, st, p);
  return DH_OK;
}

// ---- host -------------------------------------------------------------------------------------
// Query heads of a kv head are split over workgroups (each with fp32 partial dK / dV that a second kernel adds up)
// only as far as it takes to give every compute unit one workgroup: beyond that the partials cost more than the
// finer grain gives (ring step, 32 q / 8 kv heads: 4 splits 669 us, 2 splits 633 us, none 609 us).
static int pick_hsplit(int max_sk, int batch, int hq, int hk, int bn) {
  const int ratio = hq / hk;
  if (ratio == 1) return 1;
  const int64_t blocks = cdiv(max_sk, bn) * hk * batch;
  int hsplit = 1;
  for (int s = 1; s <= ratio; ++s)
    if (ratio % s == 0 && blocks * s <= 256) hsplit = s;
  return hsplit;
}

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

template <typename T, int D, int NW>
static int launch_dkv(const AttnBwdParams &p, int batch, int max_sk, hipStream_t st) {
  constexpr int BN = 32 * NW, BM = 32;
  constexpr size_t smem = 2 * 2 * BM * (D + 16) * sizeof(T) + 4 * BM * sizeof(float);
  DH_MAX_DYNAMIC_LDS_PER_DEVICE((&attn_bwd_dkv_kernel<T, D, NW>), smem);
  dim3 grid((unsigned)cdiv(max_sk, BN), (unsigned)(p.hk * p.hsplit), (unsigned)batch);
  hipLaunchKernelGGL((attn_bwd_dkv_kernel<T, D, NW>), grid, dim3(64 * NW), smem, st, p);
  return DH_OK;
}

template <typename T, int D, int NW>
static int launch_dq(const AttnBwdParams &p, int batch, hipStream_t st) {
  constexpr int BM = 32 * NW, BN = 32;
  constexpr size_t smem = 2 * BN * ((D + 16) + (D + 8)) * sizeof(T);
  DH_MAX_DYNAMIC_LDS_PER_DEVICE((&attn_bwd_dq_kernel<T, D, NW>), smem);
  dim3 grid((unsigned)cdiv(p.max_sq, BM), (unsigned)p.hq, (unsigned)batch);
  hipLaunchKernelGGL((attn_bwd_dq_kernel<T, D, NW>), grid, dim3(64 * NW), smem, st, p);
  return DH_OK;
}

template <typename T>
static int launch_delta(const void *dout, const void *out, float *delta, const float *lse, float *ld2, int64_t ld2_plane,
                        int ld2_pitch, const int32_t *cu_q, int batch, int max_sq, int hq, int d, int64_t do_stride, int64_t o_stride,
                        hipStream_t st) {
  const int nvec = d / Vec<T>::N;
  int lanes_per = 1;
  while (lanes_per < nvec && lanes_per < 64) lanes_per <<= 1;
  const int per_block = 256 / lanes_per;
  int64_t blocks = cdiv((int64_t)(ld2 ? ld2_pitch : max_sq) * hq, per_block);
  if (blocks > 256 * 16) blocks = 256 * 16;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL((attn_delta_kernel<T>), dim3((unsigned)blocks, (unsigned)batch), dim3(256), 0, st,
                     (const T *)dout, (const T *)out, delta, lse, ld2, ld2_plane, ld2_pitch, cu_q, max_sq, hq, d, lanes_per, do_stride,
                     o_stride);
  return DH_OK;
}

int attn_bwd_f32(const void *dout, const void *q, const void *k, const void *v, const float *lse, const float *delta,
                 void *dq, void *dk, void *dv, const int32_t *cu_q, const int32_t *cu_k, int batch, int max_sq,
                 int max_sk, int hq, int hk, int d, int64_t q_stride, int64_t k_stride, int64_t v_stride,
                 int64_t do_stride, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride, float scale, int causal,
                 int dq_accumulate, hipStream_t st);

constexpr int DKV_NW = 2;  // wavefronts per dK/dV workgroup (64 key rows)
// the dQ kernel's 32-key tile must divide evenly over the workgroup's threads (head dim 96 does not over 256)
constexpr bool dq_takes_4_waves(int d) { return (32 * (d / 8)) % 256 == 0; }

// Keeping dS for the dQ product costs 2 bytes per (head, query, key) of workspace, written once and read once.
// It pays where the recomputing dQ kernel runs its small-grid form (fewer than 256 workgroups of 128 query rows:
// the 8-head shard at 4096 tokens 181 -> 155 us, at 2048 tokens 95 -> 80 us); with the chip full the recomputing
// kernel is the faster one (32 heads x 4096: 610 against 669 us; 16 heads: 321 against 329), as the extra
// memory traffic then costs more than the two products saved.  Above the byte limit dS is never kept.
static std::atomic<size_t> g_ds_limit{(size_t)1280 << 20};
static std::atomic<int> g_ds_when_full{0};   // 1: keep dS also where the recomputing dQ kernel would fill the chip

// Whether the recomputing dQ kernel would fill the chip (its 128-row form).
static bool dq_big_grid(int batch, int max_sq, int hq, int causal) {
  const int64_t t = cdiv(max_sq, 128);
  return (causal ? (t + 1) / 2 : t) * hq * batch >= 256;
}

// Bytes of the dS blocks for these sizes (key count as an upper bound of the longest sequence); 0 for calls that
// never keep dS, whatever space there is (other head dims, fp32, a chip-filling recomputing kernel).
static size_t ds_bytes_wanted(int batch, int max_sq, int64_t max_sk, int hq, int d, int dtype, int causal) {
  if (dtype == DH_F32 || d != 128 || batch <= 0 || max_sq <= 0 || max_sk <= 0) return 0;
  if (dq_big_grid(batch, max_sq, hq, causal) && !g_ds_when_full.load()) return 0;
  // one block more per row than needed: rows a power of two apart would meet on the same memory channels
  const size_t nqt = 2 * (size_t)cdiv(max_sq, 64), nkb = 2 * (size_t)cdiv(max_sk, 64) + 1;
  return (size_t)batch * hq * nqt * nkb * 2048;
}

// ... and under the process-wide limit: 0 if they exceed it.
static size_t ds_bytes(int batch, int max_sq, int64_t max_sk, int hq, int d, int dtype, int causal) {
  const size_t n = ds_bytes_wanted(batch, max_sq, max_sk, hq, d, dtype, causal);
  return n <= g_ds_limit.load() ? n : 0;
}

// Workspace bytes every call of these sizes needs: delta, the lse / delta planes of the head-dim-128 kernels and the
// fp32 dK / dV partials of a split GQA group.  The dS blocks, where kept, lie behind them.
static size_t bwd_base_bytes(int64_t total_k, int batch, int max_seqlen_q, int hq, int hk, int d, int dtype) {
  const size_t sq = (size_t)(max_seqlen_q > 0 ? max_seqlen_q : 0);
  size_t n = align256((size_t)batch * hq * sq * sizeof(float));            // delta
  if (dtype != DH_F32 && d == 128) n += 2 * align256((size_t)batch * hq * ((sq + 31) / 32 * 32) * sizeof(float));
  if (dtype != DH_F32 && hk > 0 && hq / hk > 1)
    n += 2 * align256((size_t)(hq / hk) * (size_t)total_k * hk * d * sizeof(float));
  return n + 256;                                                          // the base pointer is rounded up to 256
}

}  // namespace dh

extern "C" void dh_attn_bwd_set_ds_limit(size_t bytes) { dh::g_ds_limit.store(bytes); }
extern "C" void dh_attn_bwd_set_ds_when_full(int on) { dh::g_ds_when_full.store(on ? 1 : 0); }

extern "C" size_t dh_attn_bwd_min_workspace_bytes(int64_t total_q, int64_t total_k, int batch, int max_seqlen_q, int hq,
                                                  int hk, int d, int dtype) {
  (void)total_q;
  return dh::bwd_base_bytes(total_k, batch, max_seqlen_q, hq, hk, d, dtype);
}

extern "C" size_t dh_attn_bwd_workspace_bytes(int64_t total_q, int64_t total_k, int batch, int max_seqlen_q, int hq,
                                              int hk, int d, int dtype) {
  using namespace dh;
  (void)total_q;
  // dS blocks, if a call of these sizes may keep them (causal or not is not known here: the causal grid is the smaller
  // one; the longest sequence has at most total_k keys)
  return bwd_base_bytes(total_k, batch, max_seqlen_q, hq, hk, d, dtype) +
         align256(ds_bytes(batch, max_seqlen_q, total_k, hq, d, dtype, 1));
}

static int attn_bwd_entry(const void *dout, const void *q, const void *k, const void *v, const void *out,
                          const float *lse, void *dq, void *dk, void *dv, float *delta_out, void *workspace,
                          size_t workspace_bytes, const int32_t *cu_seqlens_q, const int32_t *cu_seqlens_k, int batch,
                          int max_seqlen_q, int max_seqlen_k, int64_t total_q, int64_t total_k, int hq, int hk, int d,
                          int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t o_stride,
                          int64_t do_stride, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride,
                          float softmax_scale, int causal, int dq_accumulate, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(batch >= 0 && max_seqlen_q >= 0 && max_seqlen_k >= 0 && total_q >= 0 && total_k >= 0, "negative size");
  DH_CHECK(hq > 0 && hk > 0 && hq % hk == 0, "hq=%d must be a positive multiple of hk=%d", hq, hk);
  if (batch == 0) return DH_OK;
  DH_CHECK(dout && q && k && v && out && lse && dq && dk && dv && workspace && cu_seqlens_q && cu_seqlens_k,
           "null pointer");
  DH_CHECK(aligned16(workspace), "workspace must be 16-byte aligned");
  const size_t base_bytes = bwd_base_bytes(total_k, batch, max_seqlen_q, hq, hk, d, dtype);
  DH_CHECK(workspace_bytes >= base_bytes, "workspace of %zu bytes is smaller than the %zu bytes this call needs "
           "(dh_attn_bwd_min_workspace_bytes)", workspace_bytes, base_bytes);
  hipStream_t st = (hipStream_t)stream;
  uint8_t *ws = (uint8_t *)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  const size_t plane = align256((size_t)batch * hq * max_seqlen_q * sizeof(float));
  float *delta = delta_out ? delta_out : (float *)ws;
  ws += plane;
  float *ld2 = nullptr;
  const int ld2_pitch = (max_seqlen_q + 31) / 32 * 32;
  const size_t plane2 = align256((size_t)batch * hq * (size_t)ld2_pitch * sizeof(float));
  if (dtype != DH_F32 && d == 128) {
    ld2 = (float *)ws;
    ws += 2 * plane2;
    DH_CHECK(plane2 < (1ull << 31), "batch * heads * max_seqlen_q too large");
  }

  const int n = 16 / (int)dtype_size(dtype);
  DH_CHECK(d % n == 0 || dtype == DH_F32, "head dim %d must be a multiple of %d", d, n);
  DH_CHECK(do_stride % n == 0 && o_stride % n == 0 && aligned16(dout) && aligned16(out),
           "dout/out rows must be 16-byte aligned");
  // head dim 128 in 16 bits, two ways: with room for dS in the workspace the dK/dV kernel keeps it and dQ is one
  // product over it (delta from the delta kernel, which runs first); otherwise the dQ kernel recomputes S and dP,
  // forms delta itself and runs first.  Everything else uses the delta kernel.
  // dS is kept only if the blocks fit behind everything else in the workspace THIS call was given (and under the
  // process-wide limit); they take the tail of the workspace
  size_t dsb = ds_bytes(batch, max_seqlen_q, total_k, hq, d, dtype, causal);
  if (dsb > 0 && base_bytes + align256(dsb) > workspace_bytes) dsb = 0;
  const bool keep_ds = dsb > 0 && max_seqlen_k > 0;
  uint8_t *ds_ws = (uint8_t *)(((uintptr_t)workspace + 255) & ~(uintptr_t)255) + (base_bytes - 256);
  const bool delta_in_dq = dtype != DH_F32 && d == 128 && !keep_ds;
  if (max_seqlen_q > 0 && !delta_in_dq) {
    DH_DISPATCH_DTYPE(dtype, {
      launch_delta<T>(dout, out, delta, lse, ld2, (int64_t)(plane2 / sizeof(float)), ld2_pitch, cu_seqlens_q, batch, max_seqlen_q, hq, d,
                      do_stride, o_stride, st);
    });
  }
  if (dtype == DH_F32) {
    DH_CHECK(d > 0 && d <= 256 && d % 4 == 0, "fp32 attention needs d %% 4 == 0 and d <= 256 (got %d)", d);
    return attn_bwd_f32(dout, q, k, v, lse, delta, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, batch, max_seqlen_q,
                        max_seqlen_k, hq, hk, d, q_stride, k_stride, v_stride, do_stride, dq_stride, dk_stride,
                        dv_stride, softmax_scale, causal, dq_accumulate, st);
  }
  DH_CHECK(d == 64 || d == 96 || d == 128 || d == 192 || d == 256,
           "bf16/fp16 attention supports head dims 64, 96, 128, 192 and 256 (got %d); pad other sizes with zero columns", d);
  DH_CHECK(q_stride % 8 == 0 && k_stride % 8 == 0 && v_stride % 8 == 0 && dq_stride % 4 == 0 && dk_stride % 4 == 0 &&
               dv_stride % 4 == 0,
           "token strides must keep rows aligned");
  DH_CHECK(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(dq) && aligned16(dk) && aligned16(dv),
           "pointers must be 16-byte aligned");
  AttnBwdParams p;
  p.dout = dout; p.q = q; p.k = k; p.v = v; p.lse = lse; p.delta = delta;
  p.out = out; p.o_stride = o_stride;
  p.ld2 = ld2; p.ld2_plane = (int64_t)(plane2 / sizeof(float)); p.ld2_pitch = ld2_pitch;
  p.dq = dq; p.dk = dk; p.dv = dv;
  p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k;
  p.max_sq = max_seqlen_q; p.hq = hq; p.hk = hk;
  p.total_k = total_k;
  p.q_stride = q_stride; p.k_stride = k_stride; p.v_stride = v_stride; p.do_stride = do_stride;
  p.dq_stride = dq_stride; p.dk_stride = dk_stride; p.dv_stride = dv_stride;
  p.scale = softmax_scale;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  p.causal = causal;
  p.dq_accumulate = dq_accumulate ? 1 : 0;
  p.ds = keep_ds ? (void *)ds_ws : nullptr;
  p.ds_nqt = 2 * (int)cdiv(max_seqlen_q, 64);
  p.ds_nkb = 2 * (int)cdiv(max_seqlen_k < total_k ? max_seqlen_k : total_k, 64) + 1;
  p.hsplit = pick_hsplit(d == 128 && causal ? (max_seqlen_k + 1) / 2 : max_seqlen_k, batch, hq, hk, 32 * DKV_NW);
  p.dk_part = nullptr;
  p.dv_part = nullptr;
  if (p.hsplit > 1) {
    const size_t part = align256((size_t)(hq / hk) * (size_t)total_k * hk * d * sizeof(float));
    p.dk_part = (float *)ws;
    p.dv_part = (float *)(ws + part);
  }
  const bool small_q = cdiv(max_seqlen_q, 128) * hq * batch < 2 * 256;
  const bool big_q = dq_big_grid(batch, max_seqlen_q, hq, causal);
  DH_CHECK(k_stride < (1ll << 31) && v_stride < (1ll << 31) && q_stride < (1ll << 31) && do_stride < (1ll << 31),
           "token stride too large");
  int rc = DH_OK;
#define DH_BWD(TT, DD)                                                                         \
  do {                                                                                         \
    if (DD == 128 && max_seqlen_q > 0 && !keep_ds)                                             \
      rc = big_q ? launch_dq_d128<TT, 4, 2, 32>(p, batch, st) : launch_dq_d128<TT, 2, 4, 32>(p, batch, st); \
    if (rc == DH_OK && max_seqlen_k > 0)                                                       \
      rc = DD == 128 ? launch_dkv_d128<TT>(p, batch, max_seqlen_k, st) : launch_dkv<TT, DD, DKV_NW>(p, batch, max_seqlen_k, st); \
    if (rc == DH_OK && p.hsplit > 1 && total_k > 0) {                                          \
      int64_t blocks = cdiv(total_k * hk * (DD / 4), 256);                                     \
      if (blocks > 256 * 16) blocks = 256 * 16;                                                \
      hipLaunchKernelGGL((attn_bwd_gqa_sum_kernel<TT>), dim3((unsigned)blocks), dim3(256), 0, st, p.dk_part, \
                         p.dv_part, (TT *)dk, (TT *)dv, total_k, hk, DD, p.hsplit, dk_stride, dv_stride);    \
    }                                                                                          \
    if (rc == DH_OK && max_seqlen_q > 0 && DD != 128)                                          \
      rc = (small_q || !dq_takes_4_waves(DD)) ? launch_dq<TT, DD, 2>(p, batch, st)             \
                                              : launch_dq<TT, DD, dq_takes_4_waves(DD) ? 4 : 2>(p, batch, st); \
    if (rc == DH_OK && max_seqlen_q > 0 && DD == 128 && keep_ds) rc = launch_dq2_d128<TT>(p, batch, st); \
  } while (0)
#define DH_BWD_D(TT)                                                                            \
  do {                                                                                          \
    if (d == 128) DH_BWD(TT, 128); else if (d == 64) DH_BWD(TT, 64); else if (d == 96) DH_BWD(TT, 96); \
    else if (d == 192) DH_BWD(TT, 192); else DH_BWD(TT, 256);                                   \
  } while (0)
  if (dtype == DH_BF16) DH_BWD_D(bf16_t); else DH_BWD_D(f16_t);
#undef DH_BWD_D
#undef DH_BWD
  if (rc != DH_OK) return rc;
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_attn_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out,
                           const float *lse, void *dq, void *dk, void *dv, float *delta_out, void *workspace,
                           size_t workspace_bytes, const int32_t *cu_seqlens_q, const int32_t *cu_seqlens_k, int batch,
                           int max_seqlen_q, int max_seqlen_k, int64_t total_q, int64_t total_k, int hq, int hk, int d,
                           int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t o_stride,
                           int64_t do_stride, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride,
                           float softmax_scale, int causal, int dtype, void *stream) {
  return attn_bwd_entry(dout, q, k, v, out, lse, dq, dk, dv, delta_out, workspace, workspace_bytes, cu_seqlens_q, cu_seqlens_k, batch,
                        max_seqlen_q, max_seqlen_k, total_q, total_k, hq, hk, d, q_stride, k_stride, v_stride, o_stride,
                        do_stride, dq_stride, dk_stride, dv_stride, softmax_scale, causal, 0, dtype, stream);
}

extern "C" int dh_attn_bwd_acc(const void *dout, const void *q, const void *k, const void *v, const void *out,
                               const float *lse, void *dq, void *dk, void *dv, float *delta_out, void *workspace,
                               size_t workspace_bytes, const int32_t *cu_seqlens_q, const int32_t *cu_seqlens_k,
                               int batch, int max_seqlen_q, int max_seqlen_k, int64_t total_q, int64_t total_k, int hq,
                               int hk, int d, int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t o_stride,
                               int64_t do_stride, int64_t dq_stride, int64_t dk_stride, int64_t dv_stride,
                               float softmax_scale, int causal, int accumulate_dq, int dtype, void *stream) {
  return attn_bwd_entry(dout, q, k, v, out, lse, dq, dk, dv, delta_out, workspace, workspace_bytes, cu_seqlens_q, cu_seqlens_k, batch,
                        max_seqlen_q, max_seqlen_k, total_q, total_k, hq, hk, d, q_stride, k_stride, v_stride, o_stride,
                        do_stride, dq_stride, dk_stride, dv_stride, softmax_scale, causal, accumulate_dq, dtype, stream);
}

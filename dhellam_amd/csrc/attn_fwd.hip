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
#ifndef DH_FWD_RESCALE_LOG2
#define DH_FWD_RESCALE_LOG2 8
#endif
#ifndef DH_FWD_KAHEAD
#define DH_FWD_KAHEAD 2
#endif
#ifndef DH_FWD_LAG
#define DH_FWD_LAG true
#endif

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
      mx = pair32_max(mx);
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

  const float l_tot = pair32_sum(l_run);
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


// ---------------------------------------------------------------------------------------------
// Head dim 128, second-generation kernel.
//
// A workgroup is 8 wavefronts = RG row groups (32 query rows each) x SPLIT key/value
// splits.  Every iteration SPLIT tiles of BN keys are resident; split s works on tile
// it*SPLIT + s, so two wavefronts share each SIMD with independent instruction streams
// (one in MFMA while the other is in the softmax), and they share every K/V tile through
// LDS.  The partial (O, m, l) of the splits are combined through LDS at the end.
// K/V tiles go global -> LDS directly (16 bytes per lane, no staging registers, two
// stages); rows are unpadded 256 B and bank conflicts are avoided by an XOR swizzle of
// the 16-byte chunk index, applied on the global-address side of the copy:
//   K (read as 16 B row fragments):  chunk ^= row % 16
//   V (read with transpose loads) :  chunk ^= 4 * (row % 4) + (row / 4) % 4
// Causal work is made uniform by giving a workgroup the query tiles i and n-1-i.
// All global->LDS copies and all LDS reads of the main loop are written in assembly: the
// compiler then keeps no per-lane 64-bit pointers and inserts no waits of its own between
// copies in flight and fragment reads, and the copies are spread between the MFMAs so
// that they do not queue up behind each other.

// Every wavefront runs its P V products one tile late (V tiles live one iteration longer: three V slots
// against two K slots).  LAG: the second wavefront of every SIMD (the upper half of the workgroup) also
// delays its softmax to the start of the next iteration, so that one wavefront of a SIMD is in its
// matrix phase while the other is in its softmax instead of both competing for the same unit.
template <typename T, int RG, int SPLIT, int BN, bool LAG>
__global__ void __launch_bounds__(512) attn_fwd_d128_kernel(const AttnFwdParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int D = 128, BM = 32 * RG, NB = BN / 32, NS = BN / 16;
  static_assert(RG * SPLIT == 8, "8 wavefronts per workgroup");
  constexpr int TILE = BN * D;                    // elements of one K (or V) tile
  constexpr int SLOT = SPLIT * TILE;              // elements of one K (or V) slot: the tiles of all splits
  constexpr int SLOTB = SLOT * (int)sizeof(T);
  constexpr int BPT = BN / 4;                     // 1 KB copy blocks per tile
  static_assert(SPLIT * 2 * BPT == 64, "eight copy blocks per wavefront and iteration");
  constexpr int NV = 3;                           // V slots: read one iteration late, copied one ahead
  __shared__ __attribute__((aligned(1024))) T sAll[(2 + NV) * SLOT];   // K slots 0..1, then the V slots

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
  // causal: this workgroup owns query tiles (pair, nqt-1-pair); otherwise one tile
  int qt[2], nq;
  if (causal) {
    const int pair = px;
    if (2 * pair >= nqt) return;
    qt[0] = nqt - 1 - pair;
    qt[1] = pair;
    nq = (qt[0] == qt[1]) ? 1 : 2;
  } else {
    if (px >= nqt) return;
    qt[0] = px; qt[1] = 0;
    nq = 1;
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: copy bookkeeping stays scalar
  const int c = lane & 31, hh = lane >> 5;
  const int rg = w % RG, sp = w / RG;
  const bool lag = LAG && w >= 4;
  const T *kg = reinterpret_cast<const T *>(p.k) + (int64_t)k0 * p.k_stride + (int64_t)hkv * D;
  const T *vg = reinterpret_cast<const T *>(p.v) + (int64_t)k0 * p.v_stride + (int64_t)hkv * D;
  const uint32_t ldsK = (uint32_t)(uintptr_t)sAll, ldsV = ldsK + 2 * SLOTB;

  // ---- per-lane constants of the copy and of the fragment reads ---------------------------
  CopyLane cl0;                                    // copy: chunk slot and row inside a 4-row block
  cl0.l16 = lane & 15;
  cl0.lrow = lane >> 4;
  // The 8 copy blocks of a wavefront are 32 consecutive rows of ONE tile (K or V), so per iteration they
  // share a base that advances by 4 rows per block, and the lane offset only depends on block % 4
  // (through the swizzle).
  const int cp_tile = (w * 8) / (2 * BPT);            // which of the SPLIT resident tiles
  const int cp_v = ((w * 8) % (2 * BPT)) / BPT;       // 0: K, 1: V
  const int cp_r0 = 4 * ((w * 8) % BPT);              // first row inside the tile
  const int cp_stride = cp_v ? v_stride : k_stride;
  const T *cp_gt = cp_v ? vg : kg;
  const char *cp_g = reinterpret_cast<const char *>(cp_gt);
  const int cp_dst0 = cp_tile * TILE + cp_r0 * D;     // elements inside a slot
  const uint32_t cp_step = (uint32_t)(4 * cp_stride) * (uint32_t)sizeof(T);
  uint32_t cp_off[4];
  {
    const uint32_t rowb = (uint32_t)(cl0.lrow * cp_stride) * (uint32_t)sizeof(T);
    const uint32_t chunk = (uint32_t)(cp_v ? (cl0.l16 ^ (4 * cl0.lrow)) : (cl0.l16 ^ cl0.lrow)) << 4;
#pragma unroll
    for (int x = 0; x < 4; ++x) cp_off[x] = rowb + (chunk ^ (uint32_t)(x << (cp_v ? 4 : 6)));
  }
  // Fragment reads: byte offsets of the lane inside a K / V slot.  The swizzle XORs only bits 4..7 of an
  // address whose other low bits are fixed, so the remaining fragments of a tile are reached by XORing a
  // constant into these (K: 32 * ks; V: 64 * t) plus an immediate offset (K: 8 KB per 32 keys; V: 4 KB per 16).
  const int r = lane & 15;
  const uint32_t kb_lane = (uint32_t)(sp * TILE * (int)sizeof(T) + c * 256 + ((hh ^ (c & 15)) << 4));
  const int va_x = 4 * (r >> 2) + hh;                 // V transpose read, first four keys of a step
  const int v_lc = 2 * ((lane >> 4) & 1) + ((r & 3) >> 1);
  const uint32_t v_row = (uint32_t)(sp * TILE * (int)sizeof(T) + (4 * hh + (r >> 2)) * 256 + ((r & 3) & 1) * 8);
  const uint32_t va_lane = v_row + (uint32_t)((v_lc ^ va_x) << 4);
  const uint32_t vb_lane = v_row + 8 * 256 + (uint32_t)((v_lc ^ (va_x + 2)) << 4);   // second four keys (row + 8)

  for (int qi = 0; qi < nq; ++qi) {
    const int m0 = qt[qi] * BM;
    const int wrow0 = m0 + rg * 32;
    const int row_q = wrow0 + c;
    const int row_ld = row_q < sq ? row_q : sq - 1;
    const T *qp = reinterpret_cast<const T *>(p.q) + (int64_t)(q0 + row_ld) * p.q_stride + (int64_t)h * D;
    Frag Qf[D / 16];
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) Qf[ks] = frag_ld<T>(qp + ks * 16 + 8 * hh);

    int nk_end = sk;
    if (causal && m0 + BM < nk_end) nk_end = m0 + BM;
    const int ntiles = (nk_end + BN - 1) / BN;
    const int niter = (ntiles + SPLIT - 1) / SPLIT;
    const int n_fast = sk / (SPLIT * BN);          // iterations whose tiles lie wholly inside the keys

    floatx16 O[D / 32];
#pragma unroll
    for (int t = 0; t < D / 32; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) O[t][v] = 0.f;
    float m_run = -1e30f, l_run = 0.f;
    Frag Pb[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int j = 0; j < 8; ++j) Pb[s][j] = static_cast<T>(0.f);

    if (niter > 0 && cp_tile < ntiles)
      dma_tile32_general<T>(sAll + (cp_v ? 2 * SLOT : 0) + cp_dst0, cp_gt, cp_stride, cp_v, cp_tile * BN + cp_r0, cp_r0, sk, cl0);
    dma_wait_all();
    __syncthreads();

    // slots of iteration it: K it % 2, V it % NV
    uint32_t k_cur = ldsK, k_nxt = ldsK + SLOTB;
    int v_cur = 0, v_prev = NV - 1;
    bool act_prev = false;
    const char *cp_src = nullptr;
    uint32_t cp_dst = 0;
    bool fcopy = false;

#define DH_FWD_COPY(i)                                                                                  \
    do {                                                                                                \
      if (fcopy) {                                                                                      \
        __builtin_amdgcn_sched_barrier(0);                                                              \
        dma_block_fast(cp_src, cp_off[(i) & 3], cp_dst);                                                \
        cp_src += cp_step;                                                                              \
        cp_dst += 1024;                                                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                              \
      }                                                                                                 \
    } while (0)

    // O^T += V^T P^T for the tile in V slot `vs`; the wavefront's eight copy blocks go out between the MFMAs
    // of this phase, the first of the iteration, so that they have the rest of it to land.
    auto pv = [&](int vs) {
      uint32_t va = ldsV + (uint32_t)(vs * SLOTB) + va_lane, vb = ldsV + (uint32_t)(vs * SLOTB) + vb_lane;
      asm volatile("" : "+v"(va), "+v"(vb));     // derive the other addresses here, not ahead of the loop
      uint32_t ad[8];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        ad[2 * t] = va ^ (uint32_t)(t << 6);
        ad[2 * t + 1] = vb ^ (uint32_t)(t << 6);
      }
      short4v f[2][8];
      auto rd = [&](int st) {
        if (st == 0) lds_read_tr8<0>(f[st & 1], ad);
        else if (st == 1) lds_read_tr8<16 * 256>(f[st & 1], ad);
        else if (st == 2) lds_read_tr8<32 * 256>(f[st & 1], ad);
        else lds_read_tr8<48 * 256>(f[st & 1], ad);
      };
      rd(0);
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        short4v(&g)[8] = f[s & 1];
        if (s + 1 < NS) {
          rd(s + 1);
          lds_wait<12>(g[0], g[1], g[2], g[3]);
        } else {
          lds_wait<4>(g[0], g[1], g[2], g[3]);
        }
        O[0] = M::mma(frag_join<T>(g[0], g[1]), Pb[s], O[0]);
        O[1] = M::mma(frag_join<T>(g[2], g[3]), Pb[s], O[1]);
        if (NS == 2) { DH_FWD_COPY(4 * s); DH_FWD_COPY(4 * s + 1); }
        else DH_FWD_COPY(2 * s);
        if (s + 1 < NS) lds_wait<8>(g[4], g[5], g[6], g[7]);
        else lds_wait<0>(g[4], g[5], g[6], g[7]);
        O[2] = M::mma(frag_join<T>(g[4], g[5]), Pb[s], O[2]);
        O[3] = M::mma(frag_join<T>(g[6], g[7]), Pb[s], O[3]);
        if (NS == 2) { DH_FWD_COPY(4 * s + 2); DH_FWD_COPY(4 * s + 3); }
        else DH_FWD_COPY(2 * s + 1);
      }
    };

    // S^T = K Q^T for this wavefront's tile of the current iteration.
    floatx16 S[NB];
    auto qk = [&](uint32_t k_slot) {
      uint32_t kb = k_slot + kb_lane;
      asm volatile("" : "+v"(kb));
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) S[nb][v] = 0.f;
      // K fragments are fetched in pairs, DH_FWD_KAHEAD pairs ahead of the MFMAs that consume them.
      constexpr int NP = NB * (D / 16) / 2, AH = DH_FWD_KAHEAD;
      int4v ka[2 * (AH + 1)];
      auto issue = [&](int pr) {
        const int i = 2 * pr, nb = i / (D / 16), ks = i % (D / 16), q = 2 * (pr % (AH + 1));
        if (nb == 0) {
          lds_read128<0>(ka[q], kb ^ (uint32_t)(ks << 5));
          lds_read128<0>(ka[q + 1], kb ^ (uint32_t)((ks + 1) << 5));
        } else {
          lds_read128<32 * 256>(ka[q], kb ^ (uint32_t)(ks << 5));
          lds_read128<32 * 256>(ka[q + 1], kb ^ (uint32_t)((ks + 1) << 5));
        }
      };
#pragma unroll
      for (int pr = 0; pr < AH; ++pr) issue(pr);
#pragma unroll
      for (int pr = 0; pr < NP; ++pr) {
        const int i = 2 * pr, nb = i / (D / 16), ks = i % (D / 16), a = 2 * (pr % (AH + 1));
        if (pr + AH < NP) issue(pr + AH);
        const int newer = (pr + AH < NP ? AH : NP - 1 - pr) * 2;     // reads issued after this pair
        if (newer == 0) lds_wait<0>(ka[a], ka[a + 1]);
        else if (newer == 2) lds_wait<2>(ka[a], ka[a + 1]);
        else if (newer == 4) lds_wait<4>(ka[a], ka[a + 1]);
        else lds_wait<6>(ka[a], ka[a + 1]);
        S[nb] = M::mma(__builtin_bit_cast(Frag, ka[a]), Qf[ks], S[nb]);
        S[nb] = M::mma(__builtin_bit_cast(Frag, ka[a + 1]), Qf[ks + 1], S[nb]);
      }
    };

    // Online softmax of S (tile starting at key n0): masks, moves the running maximum when needed, leaves
    // P^T in Pb.
    auto softmax = [&](int n0) {
      const bool need_mask = (causal && n0 + BN - 1 > wrow0) || (n0 + BN > sk);
      if (need_mask) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int kv = n0 + nb * 32 + acc_row(v, hh);
            if (kv >= sk || (causal && kv > row_q)) S[nb][v] = -INFINITY;
          }
      }
      float mx = S[0][0];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, S[nb][v]);
      mx = pair32_max(mx);
      // Lazy rescale: the running maximum is only a reference point for the exponentials, so it may lag
      // the true maximum.  It is moved (and O, l rescaled) only when some row of the wavefront has grown
      // past it by more than DH_FWD_RESCALE_LOG2 binades; until then P <= 2^DH_FWD_RESCALE_LOG2, which
      // fp32 sums and 16-bit P hold without loss, and out = O / l and lse = m + log l are unchanged.
      const float m_new = fmaxf(m_run, mx);
      if (__any((m_new - m_run) * scale_log2 > (float)DH_FWD_RESCALE_LOG2)) {
        const float alpha = fast_exp2((m_run - m_new) * scale_log2);
        l_run *= alpha;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) O[t][v] *= alpha;
        m_run = m_new;
      }
      const float mc = m_run * scale_log2;
      float ps = 0.f;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        float pvv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          pvv[j] = fast_exp2(S[s >> 1][8 * (s & 1) + j] * scale_log2 - mc);
          ps += pvv[j];
        }
        Pb[s] = frag_pack<T>(pvv);
      }
      l_run += ps;
    };

    // Every wavefront runs P V one iteration late.  The first wavefront of a SIMD orders an iteration as
    // [P V of the previous tile, S of this tile | softmax of this tile], the second one (lag) as
    // [softmax of the previous tile | P V of the previous tile, S of this tile]: whenever one of them is in
    // its matrix phase the other is in its softmax.
    int n0_prev = 0;
#pragma unroll 1
    for (int it = 0; it < niter; ++it) {
      const int nit = it + 1;
      const bool copy = nit < niter && nit * SPLIT + cp_tile < ntiles;   // this wavefront's tile of the next iteration exists
      const int v_nxt = v_cur + 1 == NV ? 0 : v_cur + 1;
      fcopy = copy && nit < n_fast;
      cp_src = cp_g + (int64_t)((nit * SPLIT + cp_tile) * BN + cp_r0) * cp_stride * (int)sizeof(T);
      cp_dst = (cp_v ? ldsV + (uint32_t)(v_nxt * SLOTB) : k_nxt) + (uint32_t)(cp_dst0 * (int)sizeof(T));
      if (copy && !fcopy)
        dma_tile32_general<T>(sAll + (cp_v ? (2 + v_nxt) * SLOT : (nit & 1) * SLOT) + cp_dst0, cp_gt, cp_stride, cp_v,
                             (nit * SPLIT + cp_tile) * BN + cp_r0, cp_r0, sk, cl0);
      const int tile_g = it * SPLIT + sp;
      const int n0 = tile_g * BN;
      const bool act = tile_g < ntiles && !(causal && n0 > wrow0 + 31);

      if (lag && act_prev) softmax(n0_prev);
      if (act_prev) pv(v_prev);
      else { DH_FWD_COPY(0); DH_FWD_COPY(1); DH_FWD_COPY(2); DH_FWD_COPY(3); DH_FWD_COPY(4); DH_FWD_COPY(5); DH_FWD_COPY(6); DH_FWD_COPY(7); }
      if (act) qk(k_cur);
      if (!lag && act) softmax(n0);

      act_prev = act;
      n0_prev = n0;
      v_prev = v_cur;
      v_cur = v_nxt;
      { const uint32_t t = k_cur; k_cur = k_nxt; k_nxt = t; }
      dma_wait_all();
      __syncthreads();   // the next slots have landed, and everyone is done with the ones they replace next
    }
    fcopy = false;
    if (lag && act_prev) softmax(n0_prev);
    if (act_prev) pv(v_prev);
#undef DH_FWD_COPY
    __syncthreads();     // everyone is done with the tiles: the area is reused for the exchange below

    // ---- combine the key/value splits through LDS (fixed order: deterministic) --------------
    // O of split s > 0, row group g -> slot x = (s-1)*RG + g (16 KB each), then m and l of every slot.
    float *xo = reinterpret_cast<float *>(sAll);
    float *xml = xo + 6 * 4096;
    static_assert((SPLIT - 1) * RG <= 6, "exchange slots");
    static_assert((2 + NV) * SLOT * sizeof(T) >= (6 * 4096 + 6 * 128) * sizeof(float), "exchange area");
    if (sp > 0) {
      const int x = (sp - 1) * RG + rg;
      float *dst = xo + x * 4096;
#pragma unroll
      for (int t = 0; t < D / 32; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[(t * 16 + v) * 64 + lane] = O[t][v];
      xml[x * 128 + lane] = m_run;
      xml[x * 128 + 64 + lane] = l_run;
    }
    __syncthreads();
    if (sp == 0) {
#pragma unroll
      for (int s2 = 1; s2 < SPLIT; ++s2) {
        const int x = (s2 - 1) * RG + rg;
        const float *src = xo + x * 4096;
        const float m_o = xml[x * 128 + lane], l_o = xml[x * 128 + 64 + lane];
        const float m_new = fmaxf(m_run, m_o);
        const float a_me = fast_exp2((m_run - m_new) * scale_log2);
        const float a_o = fast_exp2((m_o - m_new) * scale_log2);
        l_run = l_run * a_me + l_o * a_o;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) O[t][v] = O[t][v] * a_me + src[(t * 16 + v) * 64 + lane] * a_o;
        m_run = m_new;
      }
      const float l_tot = pair32_sum(l_run);
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
    __syncthreads();   // the exchange area is reused by the next query tile's copies
  }
}

template <typename T, int RG, int SPLIT, int BN, bool LAG>
static int launch_attn_fwd_d128(const AttnFwdParams &p, int batch, hipStream_t st) {
  constexpr int BM = 32 * RG;
  const int nqt = (int)cdiv(p.max_sq, BM);
  dim3 grid((unsigned)((p.causal ? (nqt + 1) / 2 : nqt) * p.hq), (unsigned)batch);
  hipLaunchKernelGGL((attn_fwd_d128_kernel<T, RG, SPLIT, BN, LAG>), grid, dim3(512), 0, st, p);
  return DH_OK;
}

// fewest workgroups of 128 query rows for which the 128-row kernel is taken
#ifndef DH_FWD_128ROW_MIN_WG
#define DH_FWD_128ROW_MIN_WG 256
#endif

template <typename T, int D, int NW>
static int launch_attn_fwd(const AttnFwdParams &p, int batch, hipStream_t st) {
  constexpr int BM = 32 * NW, BN = 64;
  constexpr size_t smem = 2 * BN * ((D + 8) + (D + 32)) * sizeof(T);
  DH_MAX_DYNAMIC_LDS_PER_DEVICE((&attn_fwd_kernel<T, D, NW>), smem);
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
  DH_CHECK(d == 64 || d == 96 || d == 128 || d == 192 || d == 256,
           "bf16/fp16 attention supports head dims 64, 96, 128, 192 and 256 (got %d); pad other sizes with zero columns", d);
  DH_CHECK(q_stride % 8 == 0 && k_stride % 8 == 0 && v_stride % 8 == 0 && o_stride % 4 == 0,
           "token strides must keep rows 16-byte aligned");
  DH_CHECK(k_stride < (1ll << 31) && v_stride < (1ll << 31), "token stride too large");
  DH_CHECK(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out), "q/k/v/out must be 16-byte aligned");
  AttnFwdParams p;
  p.q = q; p.k = k; p.v = v; p.o = out; p.lse = lse;
  p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k;
  p.max_sq = max_seqlen_q; p.hq = hq; p.hk = hk;
  p.q_stride = q_stride; p.k_stride = k_stride; p.v_stride = v_stride; p.o_stride = o_stride;
  p.scale = softmax_scale;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  p.causal = causal;
  int rc;
  if (d == 128) {
    // 128-row query tiles when that still gives every CU a workgroup, else 64-row tiles.
    const int64_t wg128 = (causal ? (cdiv(max_seqlen_q, 128) + 1) / 2 : cdiv(max_seqlen_q, 128)) * hq * batch;
    const bool big = wg128 >= DH_FWD_128ROW_MIN_WG;
    if (dtype == DH_BF16) rc = big ? launch_attn_fwd_d128<bf16_t, 4, 2, 64, DH_FWD_LAG>(p, batch, st) : launch_attn_fwd_d128<bf16_t, 2, 4, 32, DH_FWD_LAG>(p, batch, st);
    else rc = big ? launch_attn_fwd_d128<f16_t, 4, 2, 64, DH_FWD_LAG>(p, batch, st) : launch_attn_fwd_d128<f16_t, 2, 4, 32, DH_FWD_LAG>(p, batch, st);
  } else {
    // Few query tiles (small batch*heads) -> smaller workgroups so the grid still covers the chip.
    const int64_t blocks128 = cdiv(max_seqlen_q, 128) * hq * batch;
    const bool small = blocks128 < 2 * 256;
#define DH_FWD_GENERIC(DD)                                                                                            \
  do {                                                                                                                \
    if (dtype == DH_BF16) rc = small ? launch_attn_fwd<bf16_t, DD, 2>(p, batch, st) : launch_attn_fwd<bf16_t, DD, 4>(p, batch, st); \
    else rc = small ? launch_attn_fwd<f16_t, DD, 2>(p, batch, st) : launch_attn_fwd<f16_t, DD, 4>(p, batch, st);      \
  } while (0)
    // the register-staged kernel, compiled per head dim (the other head dims of the reference's d <= 256 reach
    // these through zero padding in the binding, as flash_atten.cu:303-312 pads to a multiple of 8)
    if (d == 64) DH_FWD_GENERIC(64);
    else if (d == 96) DH_FWD_GENERIC(96);
    else if (d == 192) DH_FWD_GENERIC(192);
    else DH_FWD_GENERIC(256);
#undef DH_FWD_GENERIC
  }
  if (rc != DH_OK) return rc;
  DH_LAUNCH_CHECK();
  return DH_OK;
}

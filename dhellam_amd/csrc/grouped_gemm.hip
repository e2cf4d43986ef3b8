// Grouped GEMM on gfx950 MFMA (bf16/fp16 inputs, fp32 accumulate) for one
// expert-parallel rank: every local expert multiplies its own contiguous block
// of permuted rows.
//
// One template covers the three products a SwiGLU expert needs:
//   NT  c[r, n]  = sum_k a[r, k] * w[g][n, k]      forward  (both k-contiguous)
//   NN  c[r, n]  = sum_k a[r, k] * w[g][k, n]      dgrad    (w strided in k)
//   TN  c[g][m,n] = sum_r a[r, m] * b[r, n]        wgrad    (both strided in k = r)
// Two kernels.  grouped_gemm_w4_kernel (NT and NN at sizes that fill the chip): 256x256 tiles, four
// wavefronts of 128x128 with hand-placed copies, optionally one workgroup per compute unit that takes
// whole tiles in rounds and a k piece of a tile of the last round.  grouped_gemm_kernel (everything else, and TN): a workgroup is 2 x WVN wavefronts, each
// owning a (32*WM) x (32*WN) output block kept in accumulators; 64-deep k slices of both operands are
// staged in LDS through registers (two stages, one barrier per slice).  k-contiguous operands are read from LDS
// as 16-byte row fragments; k-strided operands stay row-major in LDS and are
// read with transpose loads, so no operand is ever transposed in memory.
// The product is formed as C^T (weights in the MFMA A slot) so that each lane
// ends up with runs of 4 consecutive output columns of one row: 8-byte stores.
// Group row ranges are read on the device from the offsets table.
#include "mma.h"
#include <atomic>

namespace dh {

constexpr int GG_BK = 64;
constexpr int GG_MAX_GROUPS = 64;

struct GGParams {
  const void *a, *b;
  void *c;
  const int32_t *offs;
  int groups;
  int64_t m_dim;   // TN: columns of a (= rows of c[g]); NT/NN: unused
  int64_t n_dim;   // output columns
  int64_t k_dim;   // NT/NN: reduction length; TN: unused (comes from offs)
  int64_t lda, ldb, ldc;
  int64_t b_group_stride, c_group_stride;
  int tiles_m, tiles_n;  // grid extents (tiles_m is an upper bound for NT/NN)
  int accumulate;
  int max_rows;          // rows the stacked operands hold: group ranges read from offs are cut off there
  float *ws;             // split last round: fp32 partial tiles, one per workgroup
  int zero_tail;         // NT/NN on grouped_gemm_w4_kernel: the kernel itself zeroes the rows of c past the last group
  int sk_grid;           // > 0: a split kernel of that many workgroups follows and takes the last round of tiles if it splits it
};

// Workgroup ids go round the 8 XCDs; this gives XCD x (the ids x, x + 8, ...) the x-th of 8 contiguous chunks of
// 0..n-1, so that neighbouring tiles share an L2 (a bijection for any n: the first n % 8 chunks are one longer).
__device__ __forceinline__ int gg_xcd_chunk(int id, int n) {
  const int q8 = n / 8, r8 = n % 8, x = id % 8;
  return x * q8 + (x < r8 ? x : r8) + id / 8;
}

// Tile t of the list -> (m tile, n tile): bands of 8 m tiles, m fastest inside a band, so that the 32 tiles an XCD has in
// flight are 8 x 4 and share 12 operand panels through its L2 instead of 18 + 2 (1-2 % on the FFN products).
__device__ __forceinline__ void gg_tile_of(int t, int tiles_m, int tiles_n, int &tm, int &tn) {
  constexpr int GM = 8;
  const int band = t / (GM * tiles_n), first = band * GM, gm = min(GM, tiles_m - first), in_band = t - band * GM * tiles_n;
  tm = first + in_band % gm;
  tn = in_band / gm;
}

// A group's row range as the kernels use it: relative to the first group and never past the rows the caller's
// buffers hold, whatever the offsets say (they live on the device, so the host cannot check them).
__device__ __forceinline__ int gg_clamp_row(int r, int max_rows) { return r < 0 ? 0 : (r > max_rows ? max_rows : r); }

// The groups' row ranges held one group per lane (at most 64 groups), read with ONE vector load per wavefront
// instead of a chain of scalar loads per group (0.25 us per group and tile): lane g has group g's clamped range
// and the inclusive prefix sum of the groups' 256-row tile counts.  Call with all lanes active.
struct GGGroupTable { int rb, re, incl; };
__device__ __forceinline__ GGGroupTable gg_group_table(const GGParams &p, int base, int &tiles_m) {
  const int lane = threadIdx.x & 63;
  int rb = 0, re = 0;
  if (lane < p.groups) {
    rb = gg_clamp_row(p.offs[lane] - base, p.max_rows);
    re = gg_clamp_row(p.offs[lane + 1] - base, p.max_rows);
  }
  int incl = (re - rb + 255) / 256;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int o = __shfl_up(incl, d, 64);
    if (lane >= d) incl += o;
  }
  tiles_m = __builtin_amdgcn_readlane(incl, 63);
  return GGGroupTable{rb, re, incl};
}
// The group that holds m tile tm_all (< tiles_m) of the stacked rows, its row range and the tile's index inside it.
__device__ __forceinline__ void gg_locate(const GGGroupTable &gt, int tm_all, int &g, int &rb, int &re, int &tm) {
  g = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(__ballot(gt.incl > tm_all)));
  rb = __builtin_amdgcn_readlane(gt.rb, g);
  re = __builtin_amdgcn_readlane(gt.re, g);
  tm = tm_all - (__builtin_amdgcn_readlane(gt.incl, g) - (re - rb + 255) / 256);
}

// Load one 64-deep k slice of an operand into registers.
//   KC (k-contiguous): tile [R rows][64 k]; element (row, k) at src[row * ld + k]
//   KS (k-strided)   : tile [64 k][R cols]; element (k, col) at src[k * ld + col]
template <typename T, int R, bool KSTRIDED, int NT>
struct TileLoader {
  static constexpr int VECS = R * GG_BK / 8;
  static constexpr int LPT = VECS / NT;
  static_assert(VECS % NT == 0, "tile must divide over the workgroup's threads");
  // rows: extent along the R dimension still valid (from tile origin); kext: valid k extent from this slice's origin
  // FULL: the whole slice lies inside the operand (no predication: straight-line loads).
  template <bool FULL>
  static __device__ __forceinline__ void gload(uint4 (&reg)[LPT], const T *src, int64_t ld, int rext, int kext, int tid) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int idx = tid + i * NT;
      int r, k;
      if (KSTRIDED) {
        k = idx / (R / 8);
        r = (idx % (R / 8)) * 8;
        reg[i] = (FULL || (k < kext && r < rext)) ? *reinterpret_cast<const uint4 *>(src + (int64_t)k * ld + r) : make_uint4(0, 0, 0, 0);
      } else {
        r = idx / (GG_BK / 8);
        k = (idx % (GG_BK / 8)) * 8;
        reg[i] = (FULL || (r < rext && k < kext)) ? *reinterpret_cast<const uint4 *>(src + (int64_t)r * ld + k) : make_uint4(0, 0, 0, 0);
      }
    }
  }
  static constexpr int LD = KSTRIDED ? R + 32 : GG_BK + 8;          // LDS row stride (elements)
  static constexpr int ELEMS = KSTRIDED ? GG_BK * LD : R * LD;      // LDS elements per stage
  static __device__ __forceinline__ void sstore(const uint4 (&reg)[LPT], T *dst, int tid) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int idx = tid + i * NT;
      if (KSTRIDED) {
        const int k = idx / (R / 8), r = (idx % (R / 8)) * 8;
        *reinterpret_cast<uint4 *>(dst + k * LD + r) = reg[i];
      } else {
        const int r = idx / (GG_BK / 8), k = (idx % (GG_BK / 8)) * 8;
        *reinterpret_cast<uint4 *>(dst + r * LD + k) = reg[i];
      }
    }
  }
  // Fragment for the 32 rows/cols starting at r0, k-step ks (16 values of k): slot j of lane half hh is k = 16ks + 8hh + j.
  static __device__ __forceinline__ typename Mma<T>::Frag frag(const T *tile, int r0, int ks, int lane) {
    const int c = lane & 31, hh = lane >> 5;
    if (KSTRIDED) return frag_ld_tr<T>(tile, LD, 16 * ks + 8 * hh, 16 * ks + 8 * hh + 4, r0 + 16 * ((lane >> 4) & 1), lane);
    return frag_ld<T>(tile + (r0 + c) * LD + ks * 16 + 8 * hh);
  }
};

// WM x WN: 32x32 accumulator blocks per wavefront; the workgroup is 2 x WVN wavefronts.
template <typename T, bool TA, bool TB, int WM, int WN, int WVN, bool GROUPED_OUT>
__global__ void __launch_bounds__(128 * WVN) grouped_gemm_kernel(const GGParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int BM = 64 * WM, BN = 32 * WN * WVN, NT = 128 * WVN;
  using LA = TileLoader<T, BM, TA, NT>;
  using LB = TileLoader<T, BN, TB, NT>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T *sA = reinterpret_cast<T *>(smem_raw);   // [2][LA::ELEMS]
  T *sB = sA + 2 * LA::ELEMS;                // [2][LB::ELEMS]

  // XCD-aware tile order: consecutive workgroup ids land on different XCDs, so give
  // each XCD a contiguous run of tiles; inside a run the m tile moves fastest (tiles
  // that share a weight panel are neighbours in one L2).
  const int ntiles = p.tiles_m * p.tiles_n;
  int pid = blockIdx.x;
  pid = gg_xcd_chunk(pid, ntiles);
  int tm = pid % p.tiles_m;
  const int tn = pid / p.tiles_m;

  const int base = p.offs[0];
  int g = 0, row_begin = 0, row_end = 0;
  if (GROUPED_OUT) {
    // wgrad: one full [m_dim, n_dim] output per group; blockIdx.y = group
    g = blockIdx.y;
    row_begin = gg_clamp_row(p.offs[g] - base, p.max_rows);
    row_end = gg_clamp_row(p.offs[g + 1] - base, p.max_rows);
  } else {
    bool found = false;
    for (int gi = 0; gi < p.groups; ++gi) {
      const int rb = gg_clamp_row(p.offs[gi] - base, p.max_rows), re = gg_clamp_row(p.offs[gi + 1] - base, p.max_rows);
      const int t = (re - rb + BM - 1) / BM;
      if (!found && tm < t) {
        g = gi; row_begin = rb; row_end = re; found = true;
      } else if (!found) {
        tm -= t;
      }
    }
    if (!found) return;
  }

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int c = lane & 31, hh = lane >> 5;
  const int wm = w / WVN, wn = w % WVN;
  const int n0 = tn * BN;

  // Operand origins and extents.
  const T *ag, *bg;
  int a_rext, b_rext;       // valid extent along the tile's non-k dimension
  int64_t k_total;
  if (GROUPED_OUT) {
    // a [rows, m_dim] (k = row), b [rows, n_dim]
    const int m0 = tm * BM;
    ag = reinterpret_cast<const T *>(p.a) + (int64_t)row_begin * p.lda + m0;
    bg = reinterpret_cast<const T *>(p.b) + (int64_t)row_begin * p.ldb + n0;
    a_rext = (int)(p.m_dim - m0);
    b_rext = (int)(p.n_dim - n0);
    k_total = row_end - row_begin;
  } else {
    const int m0 = row_begin + tm * BM;
    ag = reinterpret_cast<const T *>(p.a) + (int64_t)m0 * p.lda;
    a_rext = row_end - m0;
    bg = reinterpret_cast<const T *>(p.b) + (int64_t)g * p.b_group_stride + (TB ? (int64_t)n0 : (int64_t)n0 * p.ldb);
    b_rext = (int)(p.n_dim - n0);
    k_total = p.k_dim;
  }

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  uint4 ra[LA::LPT], rb[LB::LPT];
  const int nslices = (int)((k_total + GG_BK - 1) / GG_BK);
  auto gload = [&](int s) {
    const int64_t k0 = (int64_t)s * GG_BK;
    const int kext = (int)(k_total - k0 < GG_BK ? k_total - k0 : GG_BK);
    if (a_rext >= BM && b_rext >= BN && kext == GG_BK) {     // interior slice (wave-uniform test)
      LA::template gload<true>(ra, TA ? ag + k0 * p.lda : ag + k0, p.lda, a_rext, kext, tid);
      LB::template gload<true>(rb, TB ? bg + k0 * p.ldb : bg + k0, p.ldb, b_rext, kext, tid);
    } else {
      LA::template gload<false>(ra, TA ? ag + k0 * p.lda : ag + k0, p.lda, a_rext, kext, tid);
      LB::template gload<false>(rb, TB ? bg + k0 * p.ldb : bg + k0, p.ldb, b_rext, kext, tid);
    }
  };
  if (nslices > 0) {
    gload(0);
    LA::sstore(ra, sA, tid);
    LB::sstore(rb, sB, tid);
  }
  __syncthreads();

  for (int s = 0; s < nslices; ++s) {
    const int st = s & 1;
    if (s + 1 < nslices) gload(s + 1);
    const T *tA = sA + st * LA::ELEMS;
    const T *tB = sB + st * LB::ELEMS;
    // operand fragments are read one k step ahead of the MFMAs that use them
    Frag fa[2][WM], fb[2][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i) fa[0][i] = LA::frag(tA, wm * 32 * WM + 32 * i, 0, lane);
#pragma unroll
    for (int j = 0; j < WN; ++j) fb[0][j] = LB::frag(tB, wn * 32 * WN + 32 * j, 0, lane);
#pragma unroll
    for (int ks = 0; ks < GG_BK / 16; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < GG_BK / 16) {
#pragma unroll
        for (int i = 0; i < WM; ++i) fa[nxt][i] = LA::frag(tA, wm * 32 * WM + 32 * i, ks + 1, lane);
#pragma unroll
        for (int j = 0; j < WN; ++j) fb[nxt][j] = LB::frag(tB, wn * 32 * WN + 32 * j, ks + 1, lane);
      }
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) acc[i][j] = M::mma(fb[cur][j], fa[cur][i], acc[i][j]);  // C^T block: rows n, cols m
    }
    if (s + 1 < nslices) {
      LA::sstore(ra, sA + (st ^ 1) * LA::ELEMS, tid);
      LB::sstore(rb, sB + (st ^ 1) * LB::ELEMS, tid);
    }
    __syncthreads();
  }

  // Epilogue: lane owns output row (m) c of each 32x32 block and 4 consecutive columns per register quad.
  T *cg;
  int m_lim;
  if (GROUPED_OUT) {
    cg = reinterpret_cast<T *>(p.c) + (int64_t)g * p.c_group_stride + (int64_t)(tm * BM) * p.ldc + n0;
    m_lim = a_rext;
  } else {
    cg = reinterpret_cast<T *>(p.c) + (int64_t)(row_begin + tm * BM) * p.ldc + n0;
    m_lim = a_rext;
  }
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int m = wm * 32 * WM + 32 * i + c;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const floatx16 av = acc[i][j];
      if (m < m_lim) {
#pragma unroll
        for (int vb = 0; vb < 4; ++vb) {
          const int n = wn * 32 * WN + 32 * j + 8 * vb + 4 * hh;
          if (n < b_rext) {
            struct alignas(8) Q4 { T v[4]; };
            Q4 *dst = reinterpret_cast<Q4 *>(cg + (int64_t)m * p.ldc + n);
            Q4 o;
            if (p.accumulate) {
              const Q4 old = *dst;
#pragma unroll
              for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(av[4 * vb + e] + static_cast<float>(old.v[e]));
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(av[4 * vb + e]);
            }
            *dst = o;
          }
        }
      }
    }
  }
}

// ---- 256x256 tiles with ONE wavefront per SIMD: four wavefronts of 128x128 outputs ------------------------------
// The 256 accumulator registers of a wavefront live in AGPRs, and the loop is written slot by slot: after every
// MFMA exactly one LDS or memory instruction (fragment read, staging-register write to LDS, buffer load), so that
// the matrix pipe never waits for a burst of them and the LDS queue never fills.  A 64-deep k slice is loaded
// into registers THREE slices ahead (two staging sets of 16 x 16 bytes per lane), written to the LDS stage that
// is not being read during the first half of a slice, published by the slice's one barrier and read as fragments
// one k step (16) ahead of the MFMAs that use them.  Against eight wavefronts of 128x64 (two per SIMD): a third
// fewer fragment reads per MFMA, and the MFMAs of one wavefront run back to back instead of two wavefronts
// alternating on the pipe.
// Tiles in LDS: k-contiguous operands as [256 rows][64 k] with unpadded 128-byte rows, the 16-byte chunk index
// XORed with (row / 2) % 8 (conflict-free 16-byte row-fragment reads); a k-strided operand (B of the NN product,
// [k][n] row-major) as [64 k][256 n] with 512-byte rows, chunk ^= 4 (k % 4) + (k / 4) % 4 inside each 256-byte
// half row, read as fragments by LDS transpose reads.
//
// The loads are buffer loads issued from assembly: the compiler does not count them, every use of a staging
// register is ordered by a hand-written s_waitcnt vmcnt (loads return in order), and between its load and its
// LDS write a staging register is touched by nothing else (every build checks the generated assembly for this:
// check_grouped_gemm_loops in dhellam_amd/build.py).  The buffer descriptors do the edge handling: their
// length is cut at the group's (or n's) last row, so that rows past the end read as zero and no access leaves
// the operands, whatever the offsets table says.
typedef int gg_i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ gg_i32x4 gg_rsrc(const void *ptr, int64_t bytes) {
  const uint64_t a = (uint64_t)(uintptr_t)ptr;
  const uint32_t nb = bytes <= 0 ? 0u : (bytes > 0x7fffffffll ? 0x7fffffffu : (uint32_t)bytes);
  gg_i32x4 r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
  r[1] = __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu));   // stride 0: raw buffer
  r[2] = __builtin_amdgcn_readfirstlane((int)nb);
  r[3] = 0x00020000;
  return r;
}

// Stores a 256x256 tile held in the accumulator layout of grouped_gemm_w4_kernel (wavefront w = 2 wm + wn owns the
// 128x128 block (wm, wn); acc[i][j] is its 32x32 block (i, j), transposed: lane column c is output row c).
template <typename T, bool MAY_ACCUMULATE>
__device__ __forceinline__ void gg_w4_store(const floatx16 (&acc)[4][4], unsigned char *smem, const GGParams &p, T *cbase, int m0,
                                            int n0, int a_rext, int b_rext) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hh = lane >> 5;
  const int wm = w >> 1, wn = w & 1;
  // Epilogue: each wavefront passes its 128x128 block through a private LDS region, 64 rows at a time, and stores
  // whole 256-byte row segments (16 lanes a row, 4 rows per instruction).  Rows of 264 bytes: the 8-byte writes of
  // 32 lanes (32 rows, one column) fall on different banks.
  constexpr int EP = 264;
  static_assert(4 * 64 * EP <= 128 * 1024, "epilogue staging fits in the stage buffers");
  unsigned char *ep = smem + w * (64 * EP);
  T *cg = cbase + (int64_t)m0 * p.ldc + n0 + wn * 128;
  struct alignas(8) Q4 { T v[4]; };
  if (MAY_ACCUMULATE && p.accumulate) {
    // c += product with one rounding: straight from the accumulators (a lane owns output row c of each 32x32 block
    // and 4 consecutive columns per register quad)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = wm * 128 + 32 * i + c;
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int vb = 0; vb < 4; ++vb) {
          const int n = 32 * j + 8 * vb + 4 * hh;
          if (m < a_rext && wn * 128 + n < b_rext) {
            Q4 *dst = reinterpret_cast<Q4 *>(cg + (int64_t)m * p.ldc + n);
            const Q4 old = *dst;
            Q4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[i][j][4 * vb + e] + static_cast<float>(old.v[e]));
            *dst = o;
          }
        }
    }
    return;
  }
  const int er = lane >> 4, ec = lane & 15;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int i2 = 0; i2 < 2; ++i2)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const floatx16 av = acc[2 * h + i2][j];
#pragma unroll
        for (int vb = 0; vb < 4; ++vb) {
          Q4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(av[4 * vb + e]);
          *reinterpret_cast<Q4 *>(ep + (32 * i2 + c) * EP + (32 * j + 8 * vb + 4 * hh) * (int)sizeof(T)) = o;
        }
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    const int mh = wm * 128 + 64 * h;                   // first row of this half in the tile
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int r = 4 * it + er;
      const dh_u32x4 o = *reinterpret_cast<const dh_u32x4 *>(ep + r * EP + ec * 16);
      if (mh + r < a_rext && wn * 128 + 8 * ec < b_rext)
        *reinterpret_cast<dh_u32x4 *>(cg + (int64_t)(mh + r) * p.ldc + 8 * ec) = o;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
  }
}

// k pieces per tile of the last round: as many as there are workgroups per tile, each at least one slice.
__device__ __forceinline__ int gg_sk_pieces(int grid, int rem, int nsl) {
  if (rem <= 0) return 1;
  const int pc = grid / rem;
  return pc < 1 ? 1 : (pc > nsl ? (nsl > 0 ? nsl : 1) : pc);
}

// FORM 0: NT (both operands k-contiguous); 1: NN (b k-strided); 2: TN (both k-strided, k = the group's rows, one output
// per group).
template <typename T, int FORM, bool SK>
__global__ void __launch_bounds__(256) grouped_gemm_w4_kernel(const GGParams p) {
  constexpr bool BKS = FORM >= 1, AKS = FORM == 2;
  static_assert(!(AKS && SK), "the wgrad form has many tiles and a short k: it is never split");
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int BM = 256, ROWB = 128, BROWB = 512, TILEB = 256 * ROWB, STAGEB = 2 * TILEB;
  constexpr int NRD = AKS ? 16 : (BKS ? 12 : 8);        // LDS read instructions per k step
  __shared__ __attribute__((aligned(1024))) unsigned char smem[2 * STAGEB];

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hh = lane >> 5;
  const int wm = w >> 1, wn = w & 1;
  const int nsl = (int)(p.k_dim / 64);
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const uint32_t lda_b = (uint32_t)p.lda * (uint32_t)sizeof(T), ldb_b = (uint32_t)p.ldb * (uint32_t)sizeof(T);
  const int base = p.offs[0];

  // Rows of c past the last group, up to max_rows (usually none): zeroed here, a row per workgroup at a time, instead
  // of by a kernel of its own in front of this one (5 us per product).
  if constexpr (!AKS) {
    if (p.zero_tail) {
      const int first = gg_clamp_row(p.offs[p.groups] - base, p.max_rows);
      const int nv = (int)(p.n_dim / 8);
      for (int r = first + (int)blockIdx.x; r < p.max_rows; r += (int)gridDim.x) {
        T *row = reinterpret_cast<T *>(p.c) + (int64_t)r * p.ldc;
        for (int v = tid; v < nv; v += 256) *reinterpret_cast<dh_u32x4 *>(row + 8 * v) = dh_u32x4{0u, 0u, 0u, 0u};
      }
    }
  }

  // ---- copies ----------------------------------------------------------------------------------------------
  // k-contiguous tile [256 rows][64 k]: a lane copies chunk lc of rows lr + 32 i.
  // k-strided tile [64 k][256 n]: a lane copies chunk cx of k rows kr + 8 i.
  const int lc = tid & 7, lr = tid >> 3, cx = tid & 31, kr = tid >> 5;
  const uint32_t goff_a = AKS ? (uint32_t)kr * lda_b + (uint32_t)(cx * 16) : (uint32_t)lr * lda_b + (uint32_t)(lc * 16);
  const uint32_t goff_b = BKS ? (uint32_t)kr * ldb_b + (uint32_t)(cx * 16) : (uint32_t)lr * ldb_b + (uint32_t)(lc * 16);
  const uint32_t kstep_a = AKS ? 64 * lda_b : 64 * (uint32_t)sizeof(T);       // bytes from one k slice to the next
  const uint32_t kstep_b = BKS ? 64 * ldb_b : 64 * (uint32_t)sizeof(T);
  const uint32_t rstep_a = AKS ? 8 * lda_b : 32 * lda_b, rstep_b = BKS ? 8 * ldb_b : 32 * ldb_b;   // bytes from one copy of a lane to its next
  const uint32_t wr_kc = (uint32_t)(lr * ROWB + ((lc ^ ((lr >> 1) & 7)) << 4));                     // + i * 4096
  // k-strided tile: chunk XOR 4 (k % 4) + (k / 4) % 4 with k = kr + 8 i: the i part is bit 1 of the chunk for odd i
  const uint32_t wr_ks = (uint32_t)(kr * BROWB + (cx >> 4) * 256 + (((cx & 15) ^ (4 * (kr & 3) + (kr >> 2))) << 4));
  const uint32_t wr_a = AKS ? wr_ks : wr_kc, wr_b = (uint32_t)TILEB + (BKS ? wr_ks : wr_kc);

  // ---- fragment reads --------------------------------------------------------------------------------------
  const uint32_t sw = (uint32_t)((hh ^ ((c >> 1) & 7)) << 4);
  const uint32_t fa_lane = (uint32_t)((wm * 128 + c) * ROWB) + sw;                  // k step: XOR 32 ks; block i: + 4096 i
  const uint32_t fb_lane = (uint32_t)(TILEB + (wn * 128 + c) * ROWB) + sw;
  const int r16 = lane & 15;
  const int t_lc = 2 * ((lane >> 4) & 1) + ((r16 & 3) >> 1);
  const int tx = 4 * (r16 >> 2) + 2 * hh;
  const uint32_t t_row = (uint32_t)((8 * hh + (r16 >> 2)) * BROWB + ((r16 & 3) & 1) * 8);
  const uint32_t t_lo = t_row + (uint32_t)((t_lc ^ tx) << 4);                       // k rows 8 hh + 0..3 of a step
  const uint32_t t_hi = t_row + 4 * BROWB + (uint32_t)((t_lc ^ (tx + 1)) << 4);     // k rows 8 hh + 4..7
  const uint32_t tb_a = (uint32_t)(TILEB + wn * 256) + t_lo, tb_b = (uint32_t)(TILEB + wn * 256) + t_hi;   // B tile, this wavefront's 128 columns
  const uint32_t ta_a = (uint32_t)(wm * 256) + t_lo, ta_b = (uint32_t)(wm * 256) + t_hi;                   // A tile (TN)
  typedef __attribute__((address_space(3))) const Frag *lds_frag;
  typedef short4v __attribute__((address_space(3))) *lds_tr;
  typedef __attribute__((address_space(3))) gg_i32x4 *lds_w;

  // One segment: slices [s0, s1) of the tile (g, tm, tn).  part == nullptr: the segment is the whole k range and the
  // result goes to c; else the fp32 partial sums go to part (accumulator layout: 1 KB per wavefront instruction;
  // gg_split_reduce_kernel sums the pieces of a tile in k order).
  auto segment = [&](int g, int row_begin, int row_end, int tm, int tn, int s0, int s1, float *part) {
  // NT / NN: output rows m0.. of the stacked rows; TN: output rows m0.. of group g's own [m_dim, n_dim] result
  const int n0 = tn * 256, m0 = AKS ? tm * BM : row_begin + tm * BM;
  const int a_rext = AKS ? (int)(p.m_dim - m0) : row_end - m0, b_rext = (int)(p.n_dim - n0);
  const T *ag = reinterpret_cast<const T *>(p.a) + (AKS ? (int64_t)row_begin * p.lda + m0 : (int64_t)m0 * p.lda);
  const T *bg = AKS ? reinterpret_cast<const T *>(p.b) + (int64_t)row_begin * p.ldb + n0
                    : reinterpret_cast<const T *>(p.b) + (int64_t)g * p.b_group_stride + (BKS ? (int64_t)n0 : (int64_t)n0 * p.ldb);
  // One descriptor per operand, cut at the last row of the group (of n): the hardware compares the lane offset plus
  // the scalar offset with the length, so a row past the end reads as zero whichever 32-row block it is in.
  // (k-strided operands: cut at the last k row, i.e. the group's last row for TN; their tiles are whole in the
  // other direction, which the host checks)
  const gg_i32x4 rsa = AKS ? gg_rsrc(ag, (int64_t)(row_end - row_begin) * lda_b - (int64_t)m0 * (int)sizeof(T))
                           : gg_rsrc(ag, (int64_t)(a_rext < 256 ? a_rext : 256) * lda_b);
  const gg_i32x4 rsb = AKS ? gg_rsrc(bg, (int64_t)(row_end - row_begin) * ldb_b - (int64_t)n0 * (int)sizeof(T))
                     : BKS ? gg_rsrc(bg, (int64_t)p.k_dim * ldb_b - (int64_t)n0 * (int)sizeof(T))
                           : gg_rsrc(bg, (int64_t)(b_rext < 256 ? b_rext : 256) * ldb_b);
  const int cnt = s1 - s0;                              // slices of this segment
  floatx16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  gg_i32x4 stg[2][16];
  Frag fa[2][4];                                        // A fragments, k-contiguous form
  short4v fat[2][4][2];                                 // k-strided form
  Frag fbr[2][4];                                       // B fragments, k-contiguous form
  short4v fbt[2][4][2];                                 // k-strided form: the two transpose reads of a fragment

  auto gload = [&](int set, int idx, uint32_t ka, uint32_t kb) {   // idx 0..7: A, 8..15: B; ka, kb: byte offsets of the slice
    if (idx < 8) asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=&v"(stg[set][idx]) : "v"(goff_a), "s"(rsa), "s"(ka + idx * rstep_a) : "memory");
    else asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=&v"(stg[set][idx]) : "v"(goff_b), "s"(rsb), "s"(kb + (idx - 8) * rstep_b) : "memory");
  };
  // kc_w / kc_a / kc_b: the stage's lane addresses for the k-contiguous operands' writes and fragment reads, formed once
  // per slice and kept in registers (left to the compiler they are re-added in front of every LDS instruction)
  auto swrite = [&](int set, int idx, uint32_t stage, uint32_t kc_w) {  // stage: LDS byte address of the stage
    if (idx < 8 && !AKS) *(lds_w)(kc_w + idx * 4096) = stg[set][idx];
    else if (idx < 8) *(lds_w)(((stage + wr_a) ^ (uint32_t)((idx & 1) << 5)) + idx * 4096) = stg[set][idx];
    else if (!BKS) *(lds_w)(kc_w + TILEB + (idx - 8) * 4096) = stg[set][idx];
    else *(lds_w)(((stage + wr_b) ^ (uint32_t)(((idx - 8) & 1) << 5)) + (idx - 8) * 4096) = stg[set][idx];
  };
  // read r of a k step, in the order in which the MFMAs first need the data: B0 A0 B1 B2 B3 A1 A2 A3 (a k-strided
  // B fragment is two transpose reads).  abase/bbase: lane addresses of the stage with the k step applied.
  // a stage's lane addresses for k-contiguous fragment reads, and its base for the k-strided ones
  struct Bases { uint32_t kc_a, kc_b, stage; };
  auto bases_of = [&](uint32_t stage) { return Bases{stage + fa_lane, stage + fb_lane, stage}; };
  auto fread = [&](int set, int r, int ks, const Bases &ba) {
    if constexpr (!BKS) {
      constexpr int isb[8] = {1, 0, 1, 1, 1, 0, 0, 0}, blk[8] = {0, 0, 1, 2, 3, 1, 2, 3};
      if (!isb[r]) fa[set][blk[r]] = *(lds_frag)((ba.kc_a ^ (uint32_t)(ks << 5)) + blk[r] * 4096);
      else fbr[set][blk[r]] = *(lds_frag)((ba.kc_b ^ (uint32_t)(ks << 5)) + blk[r] * 4096);
    } else if constexpr (AKS) {
      // B0 A0 B1 B2 B3 A1 A2 A3, two transpose reads each
      constexpr int isb[8] = {1, 0, 1, 1, 1, 0, 0, 0}, blk[8] = {0, 0, 1, 2, 3, 1, 2, 3};
      const int f = r >> 1, half = r & 1;
      const uint32_t lane_addr = isb[f] ? (half ? tb_b : tb_a) : (half ? ta_b : ta_a);
      const short4v x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(((ba.stage + lane_addr) ^ (uint32_t)(blk[f] << 6)) + (uint32_t)(ks * 16 * BROWB)));
      if (isb[f]) fbt[set][blk[f]][half] = x;
      else fat[set][blk[f]][half] = x;
    } else {
      constexpr int kind[12] = {1, 2, 0, 1, 2, 1, 2, 1, 2, 0, 0, 0}, blk[12] = {0, 0, 0, 1, 1, 2, 2, 3, 3, 1, 2, 3};
      if (kind[r] == 0) fa[set][blk[r]] = *(lds_frag)((ba.kc_a ^ (uint32_t)(ks << 5)) + blk[r] * 4096);
      else if (kind[r] == 1)
        fbt[set][blk[r]][0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(((ba.stage + tb_a) ^ (uint32_t)(blk[r] << 6)) + (uint32_t)(ks * 16 * BROWB)));
      else
        fbt[set][blk[r]][1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(((ba.stage + tb_b) ^ (uint32_t)(blk[r] << 6)) + (uint32_t)(ks * 16 * BROWB)));
    }
  };

  // prologue: slice 0 into stage 0 (through set 0), slice 1 into set 1, slice 2 into set 0.  Loads of slices that
  // do not exist repeat the last slice (their data is written to a stage nobody reads).
  const int last = cnt > 0 ? cnt - 1 : 0;
  auto kof = [&](int s) { return (uint32_t)(s0 + (s < last ? s : last)); };
#pragma unroll
  for (int x = 0; x < 16; ++x) gload(0, x, kof(0) * kstep_a, kof(0) * kstep_b);
#pragma unroll
  for (int x = 0; x < 16; ++x) gload(1, x, kof(1) * kstep_a, kof(1) * kstep_b);
  asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
#pragma unroll
  for (int x = 0; x < 16; ++x) swrite(0, x, lds0, lds0 + wr_kc);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  // issue order of a staging set inside the loop: 0..7, 15, 8..14
#pragma unroll
  for (int x = 0; x < 8; ++x) gload(0, x, kof(2) * kstep_a, kof(2) * kstep_b);
  gload(0, 15, kof(2) * kstep_a, kof(2) * kstep_b);
#pragma unroll
  for (int x = 8; x < 15; ++x) gload(0, x, kof(2) * kstep_a, kof(2) * kstep_b);
  asm volatile("s_barrier" ::: "memory");
  {
    const Bases b0 = bases_of(lds0);
#pragma unroll
    for (int x = 0; x < NRD; ++x) fread(0, x, 0, b0);
  }

  // Slice s reads stage s % 2, writes slice s + 1 (staging set (s + 1) % 2, loaded two slices ago) into the other
  // stage during its first half and then loads slice s + 3 into the same set.
  int st = 0;
  auto slice = [&](auto xc, auto lastc, int s) {
    constexpr int X = decltype(xc)::value;              // s % 2
    constexpr bool LAST = decltype(lastc)::value;       // the last slice of an odd count: nothing to prepare
    uint32_t cur = lds0 + (uint32_t)(st * STAGEB), nxt = lds0 + (uint32_t)((st ^ 1) * STAGEB);
    const uint32_t ka = kof(s + 3) * kstep_a, kb = kof(s + 3) * kstep_b;
    asm volatile("" : "+s"(cur), "+s"(nxt));
    Bases bc = bases_of(cur), bn = bases_of(nxt);
    uint32_t wn_ = nxt + wr_kc;
    if constexpr (!AKS) asm volatile("" : "+v"(bc.kc_a), "+v"(bn.kc_a), "+v"(wn_));
    if constexpr (!BKS) asm volatile("" : "+v"(bc.kc_b), "+v"(bn.kc_b));
    // (the k-strided operands' addresses are left to the compiler: pinned, they cost more additions than they save)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int mi = 0; mi < 64; ++mi) {
      const int ks = mi >> 4, i = (mi >> 2) & 3, j = mi & 3, q = mi & 15;
      if constexpr (AKS) acc[i][j] = M::mma(frag_join<T>(fbt[ks & 1][j][0], fbt[ks & 1][j][1]), frag_join<T>(fat[ks & 1][i][0], fat[ks & 1][i][1]), acc[i][j]);
      else if constexpr (BKS) acc[i][j] = M::mma(frag_join<T>(fbt[ks & 1][j][0], fbt[ks & 1][j][1]), fa[ks & 1][i], acc[i][j]);
      else acc[i][j] = M::mma(fbr[ks & 1][j], fa[ks & 1][i], acc[i][j]);
      // fragment reads of the next k step, spread over the quarter (the last quarter: behind the barrier, from the next stage)
      if (ks < 3) {
        if (NRD == 8) { if (q % 2 == 0) fread((ks + 1) & 1, q / 2, ks + 1, bc); }
        else if (NRD == 12) { if (q % 4 != 3) fread((ks + 1) & 1, q - q / 4, ks + 1, bc); }
        else fread((ks + 1) & 1, q, ks + 1, bc);
      } else if (!LAST) {
        if (mi == 50) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (NRD == 8) {
          if (mi >= 50 && mi % 2 == 0) fread(0, (mi - 50) / 2, 0, bn);
          if (mi == 63) fread(0, 7, 0, bn);
        } else if (NRD == 12) {
          if (mi >= 50 && mi < 62) fread(0, mi - 50, 0, bn);
        } else {
          if (mi >= 50) fread(0, mi - 50, 0, bn);
          if (mi == 50) fread(0, 14, 0, bn);
          if (mi == 51) fread(0, 15, 0, bn);
        }
      }
      if (!LAST && mi < 32 && mi % 2 == 1) {            // LDS writes of slice s + 1: the older of the two sets in flight
        const int k = mi / 2;
        if (k == 0) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
        if (k == 8) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        swrite(X ^ 1, k, nxt, wn_);
      }
      if (!LAST && mi >= 33 && mi <= 61 && mi % 2 == 1) gload(X ^ 1, (mi - 33) / 2, ka, kb);
      if (!LAST && mi == 48) gload(X ^ 1, 15, ka, kb);
      __builtin_amdgcn_sched_barrier(0);
    }
    st ^= 1;
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  int s = 0;
#pragma unroll 1
  for (; s + 1 < cnt; s += 2) {
    slice(I0{}, std::false_type{}, s);
    slice(I1{}, std::false_type{}, s + 1);
  }
  // The loads of the last slices (unused data) still target the staging registers: wait for them, and keep the
  // registers reserved until then (for the compiler a load whose result nobody reads frees its register at once).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int x = 0; x < 16; ++x) asm volatile("" ::"v"(stg[0][x]), "v"(stg[1][x]));
  if (s < cnt) slice(I0{}, std::true_type{}, s);
  __syncthreads();                                      // everyone is done with the stages: they stage the output below

  if constexpr (SK) {
    // 16 bytes per lane and instruction: piece ((w * 16 + i * 4 + j) * 4 + vb) of the tile, 1 KB each
    float *dst = part + ((size_t)w * 64 * 4 + 0) * 64 + (size_t)lane * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int vb = 0; vb < 4; ++vb) {
          const floatx16 av = acc[i][j];
          const floatx4 o = {av[4 * vb], av[4 * vb + 1], av[4 * vb + 2], av[4 * vb + 3]};
          *reinterpret_cast<floatx4 *>(dst + (size_t)(((i * 4 + j) * 4 + vb) * 256)) = o;
        }
    __syncthreads();                                    // the next segment's copies reuse the stages
    return;
  }
  gg_w4_store<T, AKS>(acc, smem, p, AKS ? reinterpret_cast<T *>(p.c) + (int64_t)g * p.c_group_stride : reinterpret_cast<T *>(p.c), m0, n0, a_rext, b_rext);
    __syncthreads();                                    // the next segment's copies reuse the staging area
  };

  if constexpr (AKS) {
    // one output of tiles_m x tiles_n tiles per group (blockIdx.y); k = the group's rows, the last slice cut there
    const int ntiles = p.tiles_m * p.tiles_n;
    int pid = blockIdx.x;
    pid = gg_xcd_chunk(pid, ntiles);
    const int g = blockIdx.y;
    const int rb = gg_clamp_row(p.offs[g] - base, p.max_rows), re = gg_clamp_row(p.offs[g + 1] - base, p.max_rows);
    int tm, tn;
    gg_tile_of(pid, p.tiles_m, p.tiles_n, tm, tn);
    segment(g, rb, re, tm, tn, 0, (re - rb + 63) / 64, nullptr);
  } else if constexpr (!SK) {
    // The grid is sized for the host's upper bound of the tile count (it does not know how the rows split into
    // groups); the chunks of the XCDs are cut from the real count, so that every XCD gets its share of real tiles.
    int tiles_m;
    const GGGroupTable gt = gg_group_table(p, base, tiles_m);
    const int ntiles = tiles_m * p.tiles_n;
    int kept = ntiles;
    if (p.sk_grid > 0) {
      // the tiles past the last full round of sk_grid tiles belong to the split kernel, if it splits them
      const int full = ntiles / p.sk_grid, rem = ntiles - full * p.sk_grid;
      if (gg_sk_pieces(p.sk_grid, rem, nsl) > 1) kept = full * p.sk_grid;
    }
    if ((int)blockIdx.x >= kept) return;
    const int pid = gg_xcd_chunk((int)blockIdx.x, kept);              // (the XCDs share the tiles that are computed here)
    int tm_all, tn, g, rb, re, tm;
    gg_tile_of(pid, tiles_m, p.tiles_n, tm_all, tn);
    gg_locate(gt, tm_all, g, rb, re, tm);
    segment(g, rb, re, tm, tn, 0, nsl, nullptr);
  } else {
    // The last round of tiles, split along k.  The tiles (in the order of gg_tile_of) run in rounds of gridDim.x = the
    // number of compute units; grouped_gemm_w4_kernel<.., false> in front of this kernel takes the full rounds, one
    // workgroup per tile.  When the last round holds at most half as many tiles as there are workgroups, it is left to
    // this kernel: as many k pieces per tile as fit (workgroup w: tile w % rem, piece w / rem, so that neighbours work
    // on neighbouring tiles), summed afterwards in k order.  288 tiles on 256 compute units then take 1 1/8 tile
    // times instead of 2.  (A resident workgroup that also looped over the full rounds was 3-6 % slower on them than
    // one workgroup per tile.)
    int tiles_m;
    const GGGroupTable gt = gg_group_table(p, base, tiles_m);
    const int tiles = tiles_m * p.tiles_n;
    const int grid = (int)gridDim.x, full = tiles / grid, rem = tiles - full * grid;
    const int pieces = gg_sk_pieces(grid, rem, nsl);
    const int wg = gg_xcd_chunk((int)blockIdx.x, grid);                // neighbouring tiles on one XCD
    if (pieces == 1 || wg >= rem * pieces) return;
    const int ts = wg % rem, pc = wg / rem;
    int tm_all, tn, g, rb, re, tm;
    gg_tile_of(full * grid + ts, tiles_m, p.tiles_n, tm_all, tn);
    gg_locate(gt, tm_all, g, rb, re, tm);
    segment(g, rb, re, tm, tn, pc * nsl / pieces, (pc + 1) * nsl / pieces, p.ws + (size_t)wg * (256 * 256));
  }
}

// Sums the k pieces of the tiles of a split last round, in k order (deterministic), and stores the tiles.
// 16 workgroups per tile of that round: a wavefront takes one 32x32 block (w, i, j) of the accumulator layout,
// reads its 4 KB of every piece (1 KB per instruction) and writes 4 columns per lane and register quad.
template <typename T>
__global__ void __launch_bounds__(256) gg_split_reduce_kernel(const GGParams p, int sk_grid) {
  constexpr int BM = 256;
  const int nsl = (int)(p.k_dim / 64);
  const int base = p.offs[0];
  int tiles_m = 0;
  for (int gi = 0; gi < p.groups; ++gi)
    tiles_m += (gg_clamp_row(p.offs[gi + 1] - base, p.max_rows) - gg_clamp_row(p.offs[gi] - base, p.max_rows) + BM - 1) / BM;
  const int tiles = tiles_m * p.tiles_n, full = tiles / sk_grid, rem = tiles - full * sk_grid;
  const int ts = blockIdx.x / 16;                       // tile of the last round
  if (ts >= rem || nsl == 0) return;
  const int pieces = gg_sk_pieces(sk_grid, rem, nsl);
  if (pieces == 1) return;
  const int t = full * sk_grid + ts;
  const int tid = threadIdx.x, lane = tid & 63;
  const int blk = (blockIdx.x % 16) * 4 + (tid >> 6);   // (w * 4 + i) * 4 + j
  const int w = blk >> 4, i = (blk >> 2) & 3, j = blk & 3;
  floatx4 acc[4];
#pragma unroll
  for (int vb = 0; vb < 4; ++vb) acc[vb] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int pc = 0; pc < pieces; ++pc) {
    const float *src = p.ws + (size_t)(pc * rem + ts) * (256 * 256) + (size_t)blk * (4 * 256) + (size_t)lane * 4;
#pragma unroll
    for (int vb = 0; vb < 4; ++vb) acc[vb] += *reinterpret_cast<const floatx4 *>(src + vb * 256);
  }
  int tm, tn;
  gg_tile_of(t, tiles_m, p.tiles_n, tm, tn);
  int rb = 0, re = 0;
  for (int gi = 0; gi < p.groups; ++gi) {
    rb = gg_clamp_row(p.offs[gi] - base, p.max_rows); re = gg_clamp_row(p.offs[gi + 1] - base, p.max_rows);
    const int nt = (re - rb + BM - 1) / BM;
    if (tm < nt) break;
    tm -= nt;
  }
  const int c = lane & 31, hh = lane >> 5;
  const int m = (w >> 1) * 128 + 32 * i + c, n = (w & 1) * 128 + 32 * j + 4 * hh;    // + 8 vb
  const int m0 = rb + tm * BM, n0 = tn * 256;
  if (m0 + m >= re) return;
  T *dst = reinterpret_cast<T *>(p.c) + (int64_t)(m0 + m) * p.ldc + n0 + n;
  struct alignas(8) Q4 { T v[4]; };
#pragma unroll
  for (int vb = 0; vb < 4; ++vb)
    if (n0 + n + 8 * vb < p.n_dim) {
      Q4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[vb][e]);
      *reinterpret_cast<Q4 *>(dst + 8 * vb) = o;
    }
}

// Workspace of the split last round: one fp32 tile per workgroup of the grid.
constexpr int GG_SK_MAX_GRID = 256;
constexpr size_t GG_SK_WS_BYTES = (size_t)GG_SK_MAX_GRID * 256 * 256 * sizeof(float);

template <typename T>
static int launch_gg_w4_tn(GGParams p, hipStream_t st) {
  p.tiles_m = (int)(p.m_dim / 256);
  p.tiles_n = (int)(p.n_dim / 256);
  hipLaunchKernelGGL((grouped_gemm_w4_kernel<T, 2, false>), dim3((unsigned)(p.tiles_m * p.tiles_n), (unsigned)p.groups), dim3(256), 0, st, p);
  return DH_OK;
}

template <typename T, bool BKS>
static int launch_gg_w4(GGParams p, int64_t m_extent, void *workspace, size_t workspace_bytes, hipStream_t st) {
  p.tiles_n = (int)cdiv(p.n_dim, 256);
  p.tiles_m = (int)(cdiv(m_extent, 256) + p.groups);
  if (p.tiles_m <= 0 || p.tiles_n <= 0) return DH_OK;
  p.zero_tail = 1;
  int grid = 0;
  if (workspace != nullptr && p.k_dim >= 64) {
    int dev = 0, cus = 0;
    DH_HIP(hipGetDevice(&dev));
    DH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    grid = cus < GG_SK_MAX_GRID ? cus : GG_SK_MAX_GRID;
    if (workspace_bytes < (size_t)grid * 256 * 256 * sizeof(float)) grid = 0;
  }
  // With a workspace the last round of tiles may be split along k (decided on the device, where the tile count is
  // known): the first kernel then leaves that round to the split kernel.  When nothing is split the two extra
  // launches cost a few microseconds; a split saves up to half a tile time (45 us and more).
  p.sk_grid = grid;
  hipLaunchKernelGGL((grouped_gemm_w4_kernel<T, BKS ? 1 : 0, false>), dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(256), 0, st, p);
  if (grid > 0) {
    p.ws = reinterpret_cast<float *>(workspace);
    p.zero_tail = 0;                                    // done by the kernel above
    hipLaunchKernelGGL((grouped_gemm_w4_kernel<T, BKS ? 1 : 0, true>), dim3((unsigned)grid), dim3(256), 0, st, p);
    hipLaunchKernelGGL((gg_split_reduce_kernel<T>), dim3((unsigned)(16 * grid / 2)), dim3(256), 0, st, p, grid);   // at most grid / 2 tiles are split
  }
  return DH_OK;
}

template <typename T, bool TA, bool TB, int WM, int WN, int WVN, bool GROUPED_OUT>
static int launch_gg(GGParams p, int64_t m_extent, hipStream_t st) {
  constexpr int BM = 64 * WM, BN = 32 * WN * WVN, NT = 128 * WVN;
  using LA = TileLoader<T, BM, TA, NT>;
  using LB = TileLoader<T, BN, TB, NT>;
  constexpr size_t smem = 2 * (LA::ELEMS + LB::ELEMS) * sizeof(T);
  static_assert(smem <= 160 * 1024, "LDS budget");
  DH_MAX_DYNAMIC_LDS_PER_DEVICE((&grouped_gemm_kernel<T, TA, TB, WM, WN, WVN, GROUPED_OUT>), smem);
  p.tiles_n = (int)cdiv(p.n_dim, BN);
  p.tiles_m = GROUPED_OUT ? (int)cdiv(m_extent, BM) : (int)(cdiv(m_extent, BM) + p.groups);
  if (p.tiles_m <= 0 || p.tiles_n <= 0) return DH_OK;
  dim3 grid((unsigned)(p.tiles_m * p.tiles_n), GROUPED_OUT ? (unsigned)p.groups : 1u);
  hipLaunchKernelGGL((grouped_gemm_kernel<T, TA, TB, WM, WN, WVN, GROUPED_OUT>), grid, dim3(NT), smem, st, p);
  return DH_OK;
}

template <bool TA, bool TB, bool GROUPED_OUT>
static int dispatch_gg(const GGParams &p, int64_t m_extent, int dtype, hipStream_t st) {
  // 256x256 workgroup tiles when there is enough work to fill the chip with them, else 128x128.
  const int64_t big_tiles = cdiv(m_extent, 256) * cdiv(p.n_dim, 256) * (GROUPED_OUT ? p.groups : 1);
  const bool big = big_tiles >= 256;
  if (dtype == DH_BF16)
    return big ? launch_gg<bf16_t, TA, TB, 4, 2, 4, GROUPED_OUT>(p, m_extent, st)
               : launch_gg<bf16_t, TA, TB, 2, 2, 2, GROUPED_OUT>(p, m_extent, st);
  return big ? launch_gg<f16_t, TA, TB, 4, 2, 4, GROUPED_OUT>(p, m_extent, st)
             : launch_gg<f16_t, TA, TB, 2, 2, 2, GROUPED_OUT>(p, m_extent, st);
}

// Rows of c past the last group (up to max_rows) are zeroed, so that callers can hand over uninitialised
// memory whatever the row count turns out to be on the device: usually no row at all (a full fill of the
// output cost 45 us in front of the first expert GEMM).
__global__ void __launch_bounds__(256) gg_zero_tail_kernel(uint16_t *c, const int32_t *__restrict__ offs, int groups,
                                                           int64_t max_rows, int64_t n) {
  int64_t first = (int64_t)offs[groups] - offs[0];
  if (first < 0) first = 0;
  const int64_t nv = n / 8;                                // n is a multiple of 8 (checked by the callers)
  for (int64_t r = first + blockIdx.x; r < max_rows; r += gridDim.x)
    for (int64_t v = threadIdx.x; v < nv; v += 256) {
      Vec<uint16_t> z;
#pragma unroll
      for (int e = 0; e < 8; ++e) z.v[e] = 0;
      stg(c + r * n + v * 8, z);
    }
}

static void gg_zero_tail(void *c, const int32_t *offs, int groups, int64_t max_rows, int64_t n, hipStream_t st) {
  hipLaunchKernelGGL(gg_zero_tail_kernel, dim3(64), dim3(256), 0, st, (uint16_t *)c, offs, groups, max_rows, n);
}

static int gg_common_checks(const void *a, const void *b, void *c, const int32_t *offs, int groups, int dtype) {
  DH_CHECK(groups >= 1 && groups <= GG_MAX_GROUPS, "groups=%d must be in [1, %d]", groups, GG_MAX_GROUPS);
  DH_CHECK(dtype == DH_BF16 || dtype == DH_F16, "grouped GEMM supports bf16/fp16 (dtype %d)", dtype);
  DH_CHECK(a && b && c && offs, "null pointer");
  DH_CHECK(aligned16(a) && aligned16(b) && aligned16(c), "operands must be 16-byte aligned");
  return DH_OK;
}

}  // namespace dh

extern "C" size_t dh_grouped_gemm_workspace_bytes(void) { return dh::GG_SK_WS_BYTES; }

extern "C" int dh_grouped_gemm_nt(const void *a, const void *b, void *c, const int32_t *offs, int groups,
                                  int64_t max_rows, int64_t n, int64_t k, int dtype, void *workspace,
                                  size_t workspace_bytes, void *stream) {
  using namespace dh;
  DH_CHECK(max_rows >= 0 && max_rows < (1ll << 31) && n >= 0 && k >= 0, "size out of range");
  if (max_rows == 0 || n == 0) return DH_OK;
  int rc = gg_common_checks(a, b, c, offs, groups, dtype);
  if (rc) return rc;
  DH_CHECK(n % 8 == 0 && k % 8 == 0, "n=%lld and k=%lld must be multiples of 8", (long long)n, (long long)k);
  GGParams p{};
  p.a = a; p.b = b; p.c = c; p.offs = offs; p.groups = groups;
  p.n_dim = n; p.k_dim = k; p.lda = k; p.ldb = k; p.ldc = n;
  p.b_group_stride = n * k; p.accumulate = 0; p.max_rows = (int)max_rows;
  const bool big = cdiv(max_rows, 256) * cdiv(n, 256) >= 256;
  if (big && k % 64 == 0 && k <= (1ll << 21)) {
    rc = dtype == DH_BF16 ? launch_gg_w4<bf16_t, false>(p, max_rows, workspace, workspace_bytes, (hipStream_t)stream)
                          : launch_gg_w4<f16_t, false>(p, max_rows, workspace, workspace_bytes, (hipStream_t)stream);
  } else {
    gg_zero_tail(c, offs, groups, max_rows, n, (hipStream_t)stream);
    rc = dispatch_gg<false, false, false>(p, max_rows, dtype, (hipStream_t)stream);
  }
  if (rc) return rc;
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_grouped_gemm_nn(const void *a, const void *b, void *c, const int32_t *offs, int groups,
                                  int64_t max_rows, int64_t n, int64_t k, int dtype, void *workspace,
                                  size_t workspace_bytes, void *stream) {
  using namespace dh;
  DH_CHECK(max_rows >= 0 && max_rows < (1ll << 31) && n >= 0 && k >= 0, "size out of range");
  if (max_rows == 0 || n == 0) return DH_OK;
  int rc = gg_common_checks(a, b, c, offs, groups, dtype);
  if (rc) return rc;
  DH_CHECK(n % 8 == 0 && k % 8 == 0, "n=%lld and k=%lld must be multiples of 8", (long long)n, (long long)k);
  GGParams p{};
  p.a = a; p.b = b; p.c = c; p.offs = offs; p.groups = groups;
  p.n_dim = n; p.k_dim = k; p.lda = k; p.ldb = n; p.ldc = n;
  p.b_group_stride = n * k; p.accumulate = 0; p.max_rows = (int)max_rows;
  const bool big = cdiv(max_rows, 256) * cdiv(n, 256) >= 256;
  if (big && k % 64 == 0 && n % 256 == 0 && k <= (1ll << 21) && k * n * (int64_t)dtype_size(dtype) < (1ll << 31)) {
    rc = dtype == DH_BF16 ? launch_gg_w4<bf16_t, true>(p, max_rows, workspace, workspace_bytes, (hipStream_t)stream)
                          : launch_gg_w4<f16_t, true>(p, max_rows, workspace, workspace_bytes, (hipStream_t)stream);
  } else {
    gg_zero_tail(c, offs, groups, max_rows, n, (hipStream_t)stream);
    rc = dispatch_gg<false, true, false>(p, max_rows, dtype, (hipStream_t)stream);
  }
  if (rc) return rc;
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_grouped_gemm_tn(const void *a, const void *b, void *c, const int32_t *offs, int groups,
                                  int64_t max_rows, int64_t m, int64_t n, int accumulate, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(max_rows >= 0 && max_rows < (1ll << 31) && n >= 0 && m >= 0, "size out of range");
  if (m == 0 || n == 0) return DH_OK;
  int rc = gg_common_checks(a, b, c, offs, groups, dtype);
  if (rc) return rc;
  DH_CHECK(n % 8 == 0 && m % 8 == 0, "m=%lld and n=%lld must be multiples of 8", (long long)m, (long long)n);
  GGParams p{};
  p.a = a; p.b = b; p.c = c; p.offs = offs; p.groups = groups;
  p.m_dim = m; p.n_dim = n; p.lda = m; p.ldb = n; p.ldc = n;
  p.c_group_stride = m * n; p.accumulate = accumulate; p.max_rows = (int)max_rows;
  // whole 256x256 tiles, enough of them to fill the chip, and offsets that fit the 32-bit buffer addressing
  if (m % 256 == 0 && n % 256 == 0 && (m / 256) * (n / 256) * groups >= 256 && max_rows * (m > n ? m : n) * (int64_t)dtype_size(dtype) < (1ll << 31))
    rc = dtype == DH_BF16 ? launch_gg_w4_tn<bf16_t>(p, (hipStream_t)stream) : launch_gg_w4_tn<f16_t>(p, (hipStream_t)stream);
  else
    rc = dispatch_gg<true, true, true>(p, m, dtype, (hipStream_t)stream);
  if (rc) return rc;
  DH_LAUNCH_CHECK();
  return DH_OK;
}

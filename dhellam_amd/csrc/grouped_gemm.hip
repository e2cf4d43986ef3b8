// Grouped GEMM on gfx950 MFMA (bf16/fp16 inputs, fp32 accumulate) for one
// expert-parallel rank: every local expert multiplies its own contiguous block
// of permuted rows.
//
// One template covers the three products a SwiGLU expert needs:
//   NT  c[r, n]  = sum_k a[r, k] * w[g][n, k]      forward  (both k-contiguous)
//   NN  c[r, n]  = sum_k a[r, k] * w[g][k, n]      dgrad    (w strided in k)
//   TN  c[g][m,n] = sum_r a[r, m] * b[r, n]        wgrad    (both strided in k = r)
// A workgroup is 2 x WVN wavefronts, each owning a (32*WM) x (32*WN) output block
// kept in accumulators (256x256 tiles: 2x4 wavefronts of 128x64, two wavefronts per
// SIMD, so that one wavefront's loads, LDS stores and barrier waits overlap the other's
// MFMAs; with one wavefront per SIMD those phases simply added up); 64-deep k slices of
// both operands are staged in LDS
// (two stages, one barrier per slice).  k-contiguous operands are read from LDS
// as 16-byte row fragments; k-strided operands stay row-major in LDS and are
// read with transpose loads, so no operand is ever transposed in memory.
// The product is formed as C^T (weights in the MFMA A slot) so that each lane
// ends up with runs of 4 consecutive output columns of one row: 8-byte stores.
// Group row ranges are read on the device from the offsets table.
#include "mma.h"
#include <atomic>
#ifndef DH_GG_WVN
#define DH_GG_WVN 4
#endif
#ifndef DH_GG_CPI
#define DH_GG_CPI 2
#endif
#ifndef DH_GG_BKT
#define DH_GG_BKT 64
#endif
#ifndef DH_GG_NST
#define DH_GG_NST 2
#endif

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
};

// A group's row range as the kernels use it: relative to the first group and never past the rows the caller's
// buffers hold, whatever the offsets say (they live on the device, so the host cannot check them).
__device__ __forceinline__ int gg_clamp_row(int r, int max_rows) { return r < 0 ? 0 : (r > max_rows ? max_rows : r); }

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
  if (ntiles % 8 == 0) pid = (pid % 8) * (ntiles / 8) + pid / 8;
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

// ---- NT with direct global->LDS copies --------------------------------------------------------------
// The forward product at 256x256 tiles when K is a multiple of 64.  The register-staged kernel above
// runs its phases one after the other (wait for the global loads, store them to LDS, barrier, MFMAs):
// switching off one phase at a time showed their times simply add up.  Here the next k slice goes
// global -> LDS by assembly copies issued between the MFMAs of the current slice (no staging registers,
// no LDS stores, the wavefront never waits for its own loads before the end of the slice).
// Tiles are [256 rows][64 k] with unpadded 128-byte rows; the 16-byte chunk index is XORed with
// (row / 2) % 8, applied on the global side of the copy, which makes the 16-byte row-fragment reads
// conflict-free.  8 wavefronts = 2 (m) x 4 (n), 128x64 outputs each; wavefronts 0-3 copy the A tile
// (64 rows each), wavefronts 4-7 the B tile.
// WVN = 4: 8 wavefronts of 128x64 (two per SIMD, accumulators in VGPRs).
// BKT: k depth of a slice (64 or 32); NST: LDS stages.  The copies of slice s + NST - 1 are issued during
// slice s, so with NST > 2 a copy has more than a whole slice to land before anyone waits for it (with two
// stages the copies issued late in a slice are waited for almost at once: their latency is exposed).
// BKS: the B operand is k-strided ([k][n] row-major, the NN product).  Its tile is then [64 k][256 n] with
// 512-byte rows, copied two k rows per block with the transpose-read swizzle (chunk ^= 4 * (k % 4) +
// (k / 4) % 4 inside each 256-byte half row), and its fragments come from LDS transpose reads.
template <bool B> struct BoolC { static constexpr bool value = B; };

template <typename T, int WVN, int BKT, int NST, bool BKS>
__global__ void __launch_bounds__(128 * WVN) grouped_gemm_dma_kernel(const GGParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int BM = 256, BN = 256, WM = 4, WN = 8 / WVN, NW = 2 * WVN;
  static_assert(WVN == 4, "eight wavefronts of 128x64");
  static_assert(!BKS || BKT == 64, "the k-strided B tile is 64 k rows of 512 bytes");
  constexpr int BROWB = 256 * (int)sizeof(T);           // bytes of a row of the k-strided B tile
  constexpr int ROWB = BKT * (int)sizeof(T);            // bytes of a tile row (128 or 64)
  constexpr int CHUNKS = ROWB / 16;                     // 16-byte chunks per row
  constexpr int RP = 256 / ROWB;                        // rows per 256 bytes: the swizzle is (row / RP) % CHUNKS
  constexpr int RPB = 1024 / ROWB;                      // rows per 1 KB copy block
  constexpr int CPB = 2 * 256 / RPB / NW;               // copy blocks per wavefront and slice
  constexpr int KS = BKT / 16;                          // MFMA k steps per slice
  constexpr int DIST = NST - 1;                         // copies run this many slices ahead
  // With four stages a slice is published one slice BEFORE it is used, so its first fragments are
  // requested before the barrier that ends the previous slice (no LDS latency at the start of a slice).
  constexpr bool CROSS = NST >= 4;
  constexpr int WAITD = CROSS ? 2 : 1;                  // the barrier at the end of slice s publishes slice s + WAITD
  static_assert(!CROSS || KS % 2 == 0, "fragment sets alternate across slices");
  constexpr int TILEB = 256 * ROWB;                     // one operand tile
  constexpr int STAGEB = 2 * TILEB;                     // A tile, then B tile
  static_assert(NST * STAGEB <= 160 * 1024 && (DIST - 1) * CPB < 64, "LDS budget / wait counter range");
  __shared__ __attribute__((aligned(1024))) unsigned char smem[NST * STAGEB];

  // A contiguous run of tiles per XCD, m fastest (tiles that share a weight panel run together).
  // Cutting the grid into 4 x 8 super-tiles per XCD instead lowers the L2 miss traffic by a third
  // (measured) but is slower: the bound is not the fabric.  Running every full tile first and the groups'
  // cheap last tiles afterwards (long jobs first) is slower too, by 10 %: a last tile then re-reads from HBM
  // the weight panel that its group's full tiles shared through L2 long before.
  const int ntiles = p.tiles_m * p.tiles_n;
  int pid = blockIdx.x;
  if (ntiles % 8 == 0) pid = (pid % 8) * (ntiles / 8) + pid / 8;
  int tm = pid % p.tiles_m;
  const int tn = pid / p.tiles_m;
  const int base = p.offs[0];
  int g = 0, row_begin = 0, row_end = 0;
  {
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
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hh = lane >> 5;
  const int wm = w / WVN, wn = w % WVN;   // 2 x WVN wavefronts
  const int n0 = tn * BN, m0 = row_begin + tm * BM;
  const int a_rext = row_end - m0, b_rext = (int)(p.n_dim - n0);
  const T *ag = reinterpret_cast<const T *>(p.a) + (int64_t)m0 * p.lda;
  const T *bg = reinterpret_cast<const T *>(p.b) + (int64_t)g * p.b_group_stride + (BKS ? (int64_t)n0 : (int64_t)n0 * p.ldb);
  const int nslices = (int)(p.k_dim / BKT);
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

  // ---- copies ------------------------------------------------------------------------------------
  const int cp_b = w / (NW / 2);                        // 0: A tile, 1: B tile
  const bool cp_ks = BKS && cp_b;                       // this wavefront copies rows of the k-strided tile
  const int cp_row0 = cp_ks ? (64 / (NW / 2)) * (w % (NW / 2)) : RPB * CPB * (w % (NW / 2));
  const int cp_ld = (int)(cp_b ? p.ldb : p.lda);
  const int cp_ext = cp_ks ? 64 : (cp_b ? b_rext : a_rext);   // valid rows of the tile
  const T *cp_t = cp_b ? bg : ag;
  const char *cp_g = reinterpret_cast<const char *>(cp_t + (int64_t)cp_row0 * cp_ld);
  const uint32_t cp_dst0 = (uint32_t)(cp_b * TILEB + cp_row0 * (cp_ks ? BROWB : ROWB));
  const uint32_t cp_step = (uint32_t)((cp_ks ? 2 : RPB) * cp_ld) * (uint32_t)sizeof(T);
  const int64_t cp_slice = cp_ks ? (int64_t)64 * cp_ld * (int)sizeof(T) : (int64_t)ROWB;   // bytes from one k slice to the next
  const bool cp_fast = cp_ks || cp_row0 + RPB * CPB <= cp_ext;   // every row this wavefront copies exists
  const int lr = cp_ks ? lane >> 5 : lane / CHUNKS, lc = cp_ks ? lane & 15 : lane % CHUNKS;
  // row-fragment tiles: block i has swizzle (row / RP) % CHUNKS = (RPB / RP * (i % 2) + lr / RP) % CHUNKS (two values).
  // k-strided tile: block i holds k rows 2 i + lr, swizzle 4 * ((2 i + lr) % 4) + (i / 2) % 4, i.e. the lane part
  // lc ^ (4 lr) XOR the block constant ((i & 1) << 3) | ((i >> 1) & 3).
  uint32_t cp_off[2];
#pragma unroll
  for (int x = 0; x < 2; ++x)
    cp_off[x] = (uint32_t)(lr * cp_ld) * (uint32_t)sizeof(T) + (uint32_t)((lc ^ ((RPB / RP * x + lr / RP) % CHUNKS)) << 4);
  const uint32_t ks_base = (uint32_t)(lr * cp_ld) * (uint32_t)sizeof(T) + (uint32_t)(((lane >> 4) & 1) * 256);
  const uint32_t ks_chunk = (uint32_t)(lc ^ (4 * lr));
  auto block_off = [&](int i) -> uint32_t {
    if (cp_ks) return ks_base + ((ks_chunk ^ (uint32_t)(((i & 1) << 3) | ((i >> 1) & 3))) << 4);
    return cp_off[i & 1];
  };
  // general form (tiles at the edge of a group or of n): rows past the end re-read the last valid row
  auto copy_general = [&](uint32_t stage, int slice) {
#pragma unroll 1
    for (int i = 0; i < CPB; ++i) {
      const T *src;
      if (cp_ks) {
        const int row = cp_row0 + 2 * i + lr;
        const int f = 4 * (row & 3) + ((row >> 2) & 3);
        src = cp_t + ((int64_t)slice * 64 + row) * cp_ld + ((lane >> 4) & 1) * 128 + ((lc ^ f) * 8);
      } else {
        int row = cp_row0 + RPB * i + lr;
        const int f = (row / RP) % CHUNKS;
        row = row < cp_ext ? row : cp_ext - 1;
        src = cp_t + (int64_t)row * cp_ld + (int64_t)slice * BKT + ((lc ^ f) * 8);
      }
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                       (__attribute__((address_space(3))) void *)(smem + stage + cp_dst0 + i * 1024), 16, 0, 0);
    }
  };
  // ---- fragment reads: byte offsets inside a stage; other k steps by XOR, other 32-row blocks by + 32 rows ----
  const uint32_t sw = (uint32_t)((hh ^ ((c / RP) % CHUNKS)) << 4);
  const uint32_t fa_lane = (uint32_t)((wm * 32 * WM + c) * ROWB) + sw;            // A tile rows (m)
  const uint32_t fb_lane = (uint32_t)(TILEB + (wn * 32 * WN + c) * ROWB) + sw;    // B tile rows (n)
  // k-strided B tile: transpose reads.  A read with the lane address &tile[k0 + r / 4][n0 + 4 * (r % 4)]
  // (r = lane % 16) returns tile[k0 + 0..3][n0 + r] to the lane, so the fragment's k values 8 hh + 0..3 come
  // from a read at k0 = 8 hh and 8 hh + 4..7 from one at k0 = 8 hh + 4: the natural k order, matching the
  // row fragments of A.  t_lc: 16-byte chunk inside the 64-byte run of the 32-column block.
  const int r16 = lane & 15;
  const int t_lc = 2 * ((lane >> 4) & 1) + ((r16 & 3) >> 1);
  const int tx = 4 * (r16 >> 2) + 2 * hh;              // swizzle of k row 8 hh + r / 4; the row 4 further down has tx + 1
  const uint32_t t_row = (uint32_t)(TILEB + (8 * hh + (r16 >> 2)) * BROWB + ((r16 & 3) & 1) * 8);
  const uint32_t tb_a = t_row + (uint32_t)((t_lc ^ tx) << 4);
  const uint32_t tb_b = t_row + 4 * BROWB + (uint32_t)((t_lc ^ (tx + 1)) << 4);
  typedef __attribute__((address_space(3))) const Frag *lds_frag;
  typedef short4v __attribute__((address_space(3))) *lds_tr;
  // B fragment j of k step ks in the stage at byte offset `stage` (BKS form): the k step is an immediate offset
  auto ld_b_tr = [&](uint32_t stage, int ks, int j) -> Frag {
    const int nb = wn * WN + j;                         // 32-column block of the tile
    const uint32_t o = stage + (uint32_t)((nb >> 2) * 256);
    const uint32_t a0 = (tb_a ^ (uint32_t)((nb & 3) << 6)) + o, a1 = (tb_b ^ (uint32_t)((nb & 3) << 6)) + o;
    const short4v x0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(a0 + (uint32_t)(ks * 16 * BROWB)));
    const short4v x1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(a1 + (uint32_t)(ks * 16 * BROWB)));
    return frag_join<T>(x0, x1);
  };

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  for (int s = 0; s < DIST; ++s)
    if (s < nslices && cp_ext > 0) copy_general((uint32_t)(s * STAGEB), s);
  dma_wait_all();
  __syncthreads();

  Frag fa[2][WM], fb[2][WN];
  // fragments of k step ks of the stage whose row-fragment bases are fa_/fb_ (byte offset stage_ for the BKS form)
  // nvi: how many of this wavefront's WM 32-row blocks hold rows of the group (WM except in a group's last tile)
  auto load_frags = [&](int buf, uint32_t fa_, uint32_t fb_, uint32_t stage_, int ks, int nvi) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
      if (i < nvi) fa[buf][i] = *(lds_frag)((fa_ ^ (uint32_t)(ks << 5)) + i * 32 * ROWB);
    if (nvi > 0) {
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        if constexpr (BKS) fb[buf][j] = ld_b_tr(stage_, ks, j);
        else fb[buf][j] = *(lds_frag)((fb_ ^ (uint32_t)(ks << 5)) + j * 32 * ROWB);
      }
    }
  };
  // A group's last tile usually holds fewer than 256 rows.  Its wavefronts skip the 32-row blocks past the end
  // (fragment reads and MFMAs; the copies and barriers stay), so such a tile costs what its copies cost,
  // about a quarter of a full one, instead of a full tile's time.  The full tile keeps a branch-free loop.
  auto slices = [&](auto partial) {
  constexpr bool PARTIAL = decltype(partial)::value;
  const int nvi = PARTIAL ? min(WM, max(0, (a_rext - wm * 32 * WM + 31) >> 5)) : WM;
  if constexpr (CROSS) {
    if (nslices > 0) load_frags(0, lds0 + fa_lane, lds0 + fb_lane, lds0, 0, nvi);
  }
  int st_cur = 0, st_nxt = DIST % NST;                  // stage of slice s, stage of slice s + DIST
#pragma unroll 1
  for (int s = 0; s < nslices; ++s) {
    const uint32_t cur = (uint32_t)(st_cur * STAGEB), nxt = (uint32_t)(st_nxt * STAGEB);
    const bool copy = s + DIST < nslices && cp_ext > 0;
    const bool fcopy = copy && cp_fast;
    const char *cp_src = cp_g + (int64_t)(s + DIST) * cp_slice;
    uint32_t cp_dst = lds0 + nxt + cp_dst0;
    if (copy && !fcopy) copy_general(nxt, s + DIST);
    uint32_t fa0 = lds0 + cur + fa_lane, fb0 = lds0 + cur + fb_lane;
    const uint32_t nst1 = (uint32_t)((st_cur + 1 == NST ? 0 : st_cur + 1) * STAGEB);   // stage of slice s + 1
    uint32_t fa1 = lds0 + nst1 + fa_lane, fb1 = lds0 + nst1 + fb_lane;
    uint32_t sg0 = lds0 + cur, sg1 = lds0 + nst1;
    asm volatile("" : "+v"(fa0), "+v"(fb0), "+v"(fa1), "+v"(fb1), "+v"(sg0), "+v"(sg1));   // derive the other addresses here, not ahead of the loop
    if constexpr (!CROSS) load_frags(0, fa0, fb0, sg0, 0, nvi);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cu = ks & 1, nx = cu ^ 1;
      if (ks + 1 < KS) load_frags(nx, fa0, fb0, sg0, ks + 1, nvi);
      else if (CROSS && s + 1 < nslices) load_frags(nx, fa1, fb1, sg1, 0, nvi);   // first fragments of the next slice (already published)
#pragma unroll
      for (int i = 0; i < WM; ++i) {
#pragma unroll
        for (int j = 0; j < WN; ++j) {  // C^T block: rows n, cols m
          if (!PARTIAL || i < nvi) acc[i][j] = M::mma(fb[cu][j], fa[cu][i], acc[i][j]);
          // one 1 KB copy block after every DH_GG_CPI MFMAs until the slice's CPB blocks are out
          const int mi = (ks * WM + i) * WN + j;
          if (mi % DH_GG_CPI == DH_GG_CPI - 1 && mi / DH_GG_CPI < CPB && fcopy) {
            __builtin_amdgcn_sched_barrier(0);
            dma_block_fast(cp_src, block_off(mi / DH_GG_CPI), cp_dst);
            cp_src += cp_step;
            cp_dst += 1024;
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
    }
    // slice s + WAITD must have landed; the copies of the DIST - WAITD slices after it may still be in
    // flight (copies complete in order), unless fewer were issued (tail of k) or this wavefront uses
    // the general copies
    if (DIST > WAITD && fcopy) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DIST - WAITD) * CPB) : "memory");
    else dma_wait_all();
    st_cur = st_cur + 1 == NST ? 0 : st_cur + 1;
    st_nxt = st_nxt + 1 == NST ? 0 : st_nxt + 1;
    // A bare barrier: __syncthreads() would also wait for EVERY outstanding memory operation, i.e. drain
    // the copies that are meant to stay in flight across it.  What the barrier has to order is covered by
    // the waits above (this wavefront's copies of the slice being published) and by the fact that a
    // wavefront's fragment reads of slice s have returned before its last MFMAs of slice s were issued.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  }
  };
  if (a_rext >= BM) slices(BoolC<false>{});
  else slices(BoolC<true>{});

  // Epilogue.  A lane owns output row (m) c of each 32x32 block and 4 consecutive columns per register quad;
  // stored straight from there, an instruction would touch 32 rows with two 8-byte pieces each, and such
  // scattered partial-line stores run at a fraction of the memory system's rate (the stores were 5 % of the
  // kernel).  Each wavefront instead passes its 128x64 block through a private LDS region, 64 rows at a time,
  // and stores whole 128-byte lines: 8 adjacent lanes cover one row, 8 rows per instruction.  The stage
  // buffers are free: the barrier that ended the last slice came after every wavefront's last fragment read.
  // Rows of 136 bytes: the 8-byte writes of 32 lanes (32 rows, one column) fall on 64 different banks.
  constexpr int EP = 136;
  static_assert(NW * 64 * EP <= NST * STAGEB, "epilogue staging fits in the stage buffers");
  unsigned char *ep = smem + w * (64 * EP);
  T *cg = reinterpret_cast<T *>(p.c) + (int64_t)m0 * p.ldc + n0 + wn * 32 * WN;
  struct alignas(8) Q4 { T v[4]; };
  struct alignas(8) Q8 { Q4 lo, hi; };
  const int er = lane >> 3, ec = lane & 7;              // row inside a step of 8 rows, 16-byte chunk of the row
#pragma unroll
  for (int h = 0; h < WM / 2; ++h) {
#pragma unroll
    for (int i2 = 0; i2 < 2; ++i2) {
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        const floatx16 av = acc[2 * h + i2][j];
#pragma unroll
        for (int vb = 0; vb < 4; ++vb) {
          Q4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(av[4 * vb + e]);
          *reinterpret_cast<Q4 *>(ep + (32 * i2 + c) * EP + (32 * j + 8 * vb + 4 * hh) * (int)sizeof(T)) = o;
        }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    const int mh = wm * 32 * WM + 64 * h;               // first row of this half in the tile
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int r = 8 * it + er;
      const unsigned char *src = ep + r * EP + ec * 16;
      Q8 o;
      o.lo = *reinterpret_cast<const Q4 *>(src);
      o.hi = *reinterpret_cast<const Q4 *>(src + 8);
      const int n = wn * 32 * WN + 8 * ec;
      if (mh + r < a_rext && n < b_rext) {
        T *dst = cg + (int64_t)(mh + r) * p.ldc + 8 * ec;
        *reinterpret_cast<dh_u32x4 *>(dst) = __builtin_bit_cast(dh_u32x4, o);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
  }
}

// ---- 256x256 tiles with ONE wavefront per SIMD: four wavefronts of 128x128 outputs ------------------------------
// The 256 accumulator registers of a wavefront live in AGPRs, and the loop is written slot by slot: after every
// MFMA exactly one LDS or memory instruction (fragment read, staging-register write to LDS, buffer load), so that
// the matrix pipe never waits for a burst of them and the LDS queue never fills.  A 64-deep k slice is loaded
// into registers THREE slices ahead (two staging sets of 16 x 16 bytes per lane), written to the LDS stage that
// is not being read during the first half of a slice, published by the slice's one barrier and read as fragments
// one k step (16) ahead of the MFMAs that use them.  Against the eight-wavefront kernel above: a third fewer
// fragment reads per MFMA, MFMAs of one wavefront back to back instead of two wavefronts alternating on the pipe.
//
// The loads are buffer loads issued from assembly: the compiler does not count them, every use of a staging
// register is ordered by a hand-written s_waitcnt vmcnt (loads return in order), and between its load and its
// LDS write a staging register is touched by nothing else.  The buffer descriptors do the edge handling: one per
// 32-row block of a tile, its length cut at the group's (or n's) last row, so that rows past the end read as
// zero and no access leaves the operands, whatever the offsets table says.
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

template <typename T, bool BKS>
__global__ void __launch_bounds__(256) grouped_gemm_w4_kernel(const GGParams p) {
  using M = Mma<T>;
  using Frag = typename M::Frag;
  constexpr int BM = 256, ROWB = 128, BROWB = 512, TILEB = 256 * ROWB, STAGEB = 2 * TILEB;
  constexpr int NRD = BKS ? 12 : 8;                     // LDS read instructions per k step
  __shared__ __attribute__((aligned(1024))) unsigned char smem[2 * STAGEB];

  const int ntiles = p.tiles_m * p.tiles_n;
  int pid = blockIdx.x;
  if (ntiles % 8 == 0) pid = (pid % 8) * (ntiles / 8) + pid / 8;
  int tm = pid % p.tiles_m;
  const int tn = pid / p.tiles_m;
  const int base = p.offs[0];
  int g = 0, row_begin = 0, row_end = 0;
  {
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
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hh = lane >> 5;
  const int wm = w >> 1, wn = w & 1;
  const int n0 = tn * 256, m0 = row_begin + tm * BM;
  const int a_rext = row_end - m0, b_rext = (int)(p.n_dim - n0);
  const T *ag = reinterpret_cast<const T *>(p.a) + (int64_t)m0 * p.lda;
  const T *bg = reinterpret_cast<const T *>(p.b) + (int64_t)g * p.b_group_stride + (BKS ? (int64_t)n0 : (int64_t)n0 * p.ldb);
  const int nsl = (int)(p.k_dim / 64);
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const uint32_t lda_b = (uint32_t)p.lda * (uint32_t)sizeof(T), ldb_b = (uint32_t)p.ldb * (uint32_t)sizeof(T);

  // ---- copies ----------------------------------------------------------------------------------------------
  // k-contiguous tile [256 rows][64 k]: a lane copies chunk lc of rows lr + 32 i; descriptor i starts at row 32 i.
  // k-strided tile [64 k][256 n]: a lane copies chunk cx of k rows kr + 8 i; descriptor i starts at k row 8 i.
  const int lc = tid & 7, lr = tid >> 3, cx = tid & 31, kr = tid >> 5;
  gg_i32x4 rsa[8], rsb[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    rsa[i] = gg_rsrc(ag + (int64_t)(32 * i) * p.lda, (int64_t)(a_rext - 32 * i) * lda_b);
    if (BKS) rsb[i] = gg_rsrc(bg + (int64_t)(8 * i) * p.ldb, 0x7fffffffll);
    else rsb[i] = gg_rsrc(bg + (int64_t)(32 * i) * p.ldb, (int64_t)(b_rext - 32 * i) * ldb_b);
  }
  const uint32_t goff_a = (uint32_t)lr * lda_b + (uint32_t)(lc * 16);
  const uint32_t goff_b = BKS ? (uint32_t)kr * ldb_b + (uint32_t)(cx * 16) : (uint32_t)lr * ldb_b + (uint32_t)(lc * 16);
  const uint32_t kstep_a = 64 * (uint32_t)sizeof(T);                          // bytes from one k slice to the next
  const uint32_t kstep_b = BKS ? 64 * ldb_b : 64 * (uint32_t)sizeof(T);
  const uint32_t wr_a = (uint32_t)(lr * ROWB + ((lc ^ ((lr >> 1) & 7)) << 4));                      // + i * 4096
  // k-strided tile: chunk XOR 4 (k % 4) + (k / 4) % 4 with k = kr + 8 i: the i part is bit 1 of the chunk for odd i
  const uint32_t wr_b = BKS ? (uint32_t)(TILEB + kr * BROWB + (cx >> 4) * 256 + (((cx & 15) ^ (4 * (kr & 3) + (kr >> 2))) << 4))
                            : (uint32_t)TILEB + wr_a;

  // ---- fragment reads --------------------------------------------------------------------------------------
  const uint32_t sw = (uint32_t)((hh ^ ((c >> 1) & 7)) << 4);
  const uint32_t fa_lane = (uint32_t)((wm * 128 + c) * ROWB) + sw;                  // k step: XOR 32 ks; block i: + 4096 i
  const uint32_t fb_lane = (uint32_t)(TILEB + (wn * 128 + c) * ROWB) + sw;
  const int r16 = lane & 15;
  const int t_lc = 2 * ((lane >> 4) & 1) + ((r16 & 3) >> 1);
  const int tx = 4 * (r16 >> 2) + 2 * hh;
  const uint32_t t_row = (uint32_t)(TILEB + wn * 256 + (8 * hh + (r16 >> 2)) * BROWB + ((r16 & 3) & 1) * 8);
  const uint32_t tb_a = t_row + (uint32_t)((t_lc ^ tx) << 4);                       // k rows 8 hh + 0..3 of a step
  const uint32_t tb_b = t_row + 4 * BROWB + (uint32_t)((t_lc ^ (tx + 1)) << 4);     // k rows 8 hh + 4..7
  typedef __attribute__((address_space(3))) const Frag *lds_frag;
  typedef short4v __attribute__((address_space(3))) *lds_tr;
  typedef __attribute__((address_space(3))) gg_i32x4 *lds_w;

  floatx16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  gg_i32x4 stg[2][16];
  Frag fa[2][4];
  Frag fbr[2][4];                                       // B fragments, k-contiguous form
  short4v fbt[2][4][2];                                 // k-strided form: the two transpose reads of a fragment

  auto gload = [&](int set, int idx, uint32_t ka, uint32_t kb) {   // idx 0..7: A, 8..15: B; ka, kb: byte offsets of the slice
    if (idx < 8) asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=&v"(stg[set][idx]) : "v"(goff_a), "s"(rsa[idx]), "s"(ka) : "memory");
    else asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=&v"(stg[set][idx]) : "v"(goff_b), "s"(rsb[idx - 8]), "s"(kb) : "memory");
  };
  auto swrite = [&](int set, int idx, uint32_t stage) {  // stage: LDS byte address of the stage
    if (idx < 8) *(lds_w)(stage + wr_a + idx * 4096) = stg[set][idx];
    else if (!BKS) *(lds_w)(stage + wr_b + (idx - 8) * 4096) = stg[set][idx];
    else *(lds_w)(((stage + wr_b) ^ (uint32_t)(((idx - 8) & 1) << 5)) + (idx - 8) * 4096) = stg[set][idx];
  };
  // read r of a k step, in the order in which the MFMAs first need the data: B0 A0 B1 B2 B3 A1 A2 A3 (a k-strided
  // B fragment is two transpose reads).  abase/bbase: lane addresses of the stage with the k step applied.
  auto fread = [&](int set, int r, uint32_t stage, int ks) {
    if constexpr (!BKS) {
      constexpr int isb[8] = {1, 0, 1, 1, 1, 0, 0, 0}, blk[8] = {0, 0, 1, 2, 3, 1, 2, 3};
      if (!isb[r]) fa[set][blk[r]] = *(lds_frag)(((stage + fa_lane) ^ (uint32_t)(ks << 5)) + blk[r] * 4096);
      else fbr[set][blk[r]] = *(lds_frag)(((stage + fb_lane) ^ (uint32_t)(ks << 5)) + blk[r] * 4096);
    } else {
      constexpr int kind[12] = {1, 2, 0, 1, 2, 1, 2, 1, 2, 0, 0, 0}, blk[12] = {0, 0, 0, 1, 1, 2, 2, 3, 3, 1, 2, 3};
      if (kind[r] == 0) fa[set][blk[r]] = *(lds_frag)(((stage + fa_lane) ^ (uint32_t)(ks << 5)) + blk[r] * 4096);
      else if (kind[r] == 1)
        fbt[set][blk[r]][0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(((stage + tb_a) ^ (uint32_t)(blk[r] << 6)) + (uint32_t)(ks * 16 * BROWB)));
      else
        fbt[set][blk[r]][1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(((stage + tb_b) ^ (uint32_t)(blk[r] << 6)) + (uint32_t)(ks * 16 * BROWB)));
    }
  };

  // prologue: slice 0 into stage 0 (through set 0), slice 1 into set 1, slice 2 into set 0.  Loads of slices that
  // do not exist repeat the last slice (their data is written to a stage nobody reads).
  const int last = nsl > 0 ? nsl - 1 : 0;
  auto kof = [&](int s) { return (uint32_t)(s < last ? s : last); };
#pragma unroll
  for (int x = 0; x < 16; ++x) gload(0, x, 0, 0);
#pragma unroll
  for (int x = 0; x < 16; ++x) gload(1, x, kof(1) * kstep_a, kof(1) * kstep_b);
  asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
#pragma unroll
  for (int x = 0; x < 16; ++x) swrite(0, x, lds0);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  // issue order of a staging set inside the loop: 0..7, 15, 8..14
#pragma unroll
  for (int x = 0; x < 8; ++x) gload(0, x, kof(2) * kstep_a, kof(2) * kstep_b);
  gload(0, 15, kof(2) * kstep_a, kof(2) * kstep_b);
#pragma unroll
  for (int x = 8; x < 15; ++x) gload(0, x, kof(2) * kstep_a, kof(2) * kstep_b);
  asm volatile("s_barrier" ::: "memory");
#pragma unroll
  for (int x = 0; x < NRD; ++x) fread(0, x, lds0, 0);

  // Slice s reads stage s % 2, writes slice s + 1 (staging set (s + 1) % 2, loaded two slices ago) into the other
  // stage during its first half and then loads slice s + 3 into the same set.
  int st = 0;
  auto slice = [&](auto xc, auto lastc, int s) {
    constexpr int X = decltype(xc)::value;              // s % 2
    constexpr bool LAST = decltype(lastc)::value;       // the last slice of an odd count: nothing to prepare
    uint32_t cur = lds0 + (uint32_t)(st * STAGEB), nxt = lds0 + (uint32_t)((st ^ 1) * STAGEB);
    const uint32_t ka = kof(s + 3) * kstep_a, kb = kof(s + 3) * kstep_b;
    asm volatile("" : "+s"(cur), "+s"(nxt));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int mi = 0; mi < 64; ++mi) {
      const int ks = mi >> 4, i = (mi >> 2) & 3, j = mi & 3, q = mi & 15;
      if constexpr (BKS) acc[i][j] = M::mma(frag_join<T>(fbt[ks & 1][j][0], fbt[ks & 1][j][1]), fa[ks & 1][i], acc[i][j]);
      else acc[i][j] = M::mma(fbr[ks & 1][j], fa[ks & 1][i], acc[i][j]);
      // fragment reads of the next k step, spread over the quarter (the last quarter: behind the barrier, from the next stage)
      if (ks < 3) {
        if (NRD == 8) { if (q % 2 == 0) fread((ks + 1) & 1, q / 2, cur, ks + 1); }
        else { if (q % 4 != 3) fread((ks + 1) & 1, q - q / 4, cur, ks + 1); }
      } else if (!LAST) {
        if (mi == 50) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (NRD == 8) {
          if (mi >= 50 && mi % 2 == 0) fread(0, (mi - 50) / 2, nxt, 0);
          if (mi == 63) fread(0, 7, nxt, 0);
        } else {
          if (mi >= 50 && mi < 62) fread(0, mi - 50, nxt, 0);
        }
      }
      if (!LAST && mi < 32 && mi % 2 == 1) {            // LDS writes of slice s + 1: the older of the two sets in flight
        const int k = mi / 2;
        if (k == 0) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
        if (k == 8) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        swrite(X ^ 1, k, nxt);
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
  for (; s + 1 < nsl; s += 2) {
    slice(I0{}, std::false_type{}, s);
    slice(I1{}, std::false_type{}, s + 1);
  }
  // The loads of the last slices (unused data) still target the staging registers: wait for them, and keep the
  // registers reserved until then (for the compiler a load whose result nobody reads frees its register at once).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int x = 0; x < 16; ++x) asm volatile("" ::"v"(stg[0][x]), "v"(stg[1][x]));
  if (s < nsl) slice(I0{}, std::true_type{}, s);
  __syncthreads();                                      // everyone is done with the stages: they stage the output below

  // Epilogue: each wavefront passes its 128x128 block through a private LDS region, 64 rows at a time, and stores
  // whole 256-byte row segments (16 lanes a row, 4 rows per instruction).  Rows of 264 bytes: the 8-byte writes of
  // 32 lanes (32 rows, one column) fall on different banks.
  constexpr int EP = 264;
  static_assert(4 * 64 * EP <= 2 * STAGEB, "epilogue staging fits in the stage buffers");
  unsigned char *ep = smem + w * (64 * EP);
  T *cg = reinterpret_cast<T *>(p.c) + (int64_t)m0 * p.ldc + n0 + wn * 128;
  struct alignas(8) Q4 { T v[4]; };
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

template <typename T, bool BKS>
static int launch_gg_w4(GGParams p, int64_t m_extent, hipStream_t st) {
  p.tiles_n = (int)cdiv(p.n_dim, 256);
  p.tiles_m = (int)(cdiv(m_extent, 256) + p.groups);
  if (p.tiles_m <= 0 || p.tiles_n <= 0) return DH_OK;
  hipLaunchKernelGGL((grouped_gemm_w4_kernel<T, BKS>), dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(256), 0, st, p);
  return DH_OK;
}

template <typename T, int WVN, int BKT, int NST, bool BKS>
static int launch_gg_dma(GGParams p, int64_t m_extent, hipStream_t st) {
  p.tiles_n = (int)cdiv(p.n_dim, 256);
  p.tiles_m = (int)(cdiv(m_extent, 256) + p.groups);
  if (p.tiles_m <= 0 || p.tiles_n <= 0) return DH_OK;
  hipLaunchKernelGGL((grouped_gemm_dma_kernel<T, WVN, BKT, NST, BKS>), dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(128 * WVN), 0, st, p);
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

extern "C" int dh_grouped_gemm_nt(const void *a, const void *b, void *c, const int32_t *offs, int groups,
                                  int64_t max_rows, int64_t n, int64_t k, int dtype, void *stream) {
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
  gg_zero_tail(c, offs, groups, max_rows, n, (hipStream_t)stream);
  const bool big = cdiv(max_rows, 256) * cdiv(n, 256) >= 256;
  if (big && k % 64 == 0 && k <= (1ll << 21))
    rc = dtype == DH_BF16 ? launch_gg_w4<bf16_t, false>(p, max_rows, (hipStream_t)stream)
                          : launch_gg_w4<f16_t, false>(p, max_rows, (hipStream_t)stream);
  else if (big && k % 64 == 0 && k < (1ll << 30))
    rc = dtype == DH_BF16 ? launch_gg_dma<bf16_t, DH_GG_WVN, DH_GG_BKT, DH_GG_NST, false>(p, max_rows, (hipStream_t)stream)
                          : launch_gg_dma<f16_t, DH_GG_WVN, DH_GG_BKT, DH_GG_NST, false>(p, max_rows, (hipStream_t)stream);
  else
    rc = dispatch_gg<false, false, false>(p, max_rows, dtype, (hipStream_t)stream);
  if (rc) return rc;
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_grouped_gemm_nn(const void *a, const void *b, void *c, const int32_t *offs, int groups,
                                  int64_t max_rows, int64_t n, int64_t k, int dtype, void *stream) {
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
  gg_zero_tail(c, offs, groups, max_rows, n, (hipStream_t)stream);
  const bool big = cdiv(max_rows, 256) * cdiv(n, 256) >= 256;
  if (big && k % 64 == 0 && n % 256 == 0 && k <= (1ll << 21) && k * n * (int64_t)dtype_size(dtype) < (1ll << 31))
    rc = dtype == DH_BF16 ? launch_gg_w4<bf16_t, true>(p, max_rows, (hipStream_t)stream)
                          : launch_gg_w4<f16_t, true>(p, max_rows, (hipStream_t)stream);
  else if (big && k % 64 == 0 && n % 256 == 0 && DH_GG_BKT == 64 && n * (int64_t)dtype_size(dtype) < (1ll << 30))
    rc = dtype == DH_BF16 ? launch_gg_dma<bf16_t, DH_GG_WVN, 64, DH_GG_NST, true>(p, max_rows, (hipStream_t)stream)
                          : launch_gg_dma<f16_t, DH_GG_WVN, 64, DH_GG_NST, true>(p, max_rows, (hipStream_t)stream);
  else
    rc = dispatch_gg<false, true, false>(p, max_rows, dtype, (hipStream_t)stream);
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
  rc = dispatch_gg<true, true, true>(p, m, dtype, (hipStream_t)stream);
  if (rc) return rc;
  DH_LAUNCH_CHECK();
  return DH_OK;
}

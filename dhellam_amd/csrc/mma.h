// MFMA building blocks for gfx950 (CDNA4), 16-bit inputs, fp32 accumulate.
//
// One "atom" is v_mfma_f32_32x32x16_{bf16,f16}: D[32x32] += A[32x16] * B[16x32].
// Register layout for wave lane l (c = l % 32, h = l / 32):
//   A operand: 8 values A[row = c][k = 8h + j], j = 0..7
//   B operand: 8 values B[k = 8h + j][col = c]
//   D: 16 floats, D[row = 8*(v/4) + 4h + v%4][col = c], v = 0..15
// Because A and B index k the same way, any consistent relabelling of k between
// the two operands leaves the product unchanged; the attention kernels use that
// to feed an accumulator (whose rows are 8*(v/4)+4h+v%4) straight back in as an
// operand without a shuffle.
//
// ds_read_b64_tr_b16 (LDS transpose read): within each group of 16 lanes, lane
// r supplies the address of 4 consecutive 16-bit values M[r][0..3]; lane i
// receives M[i/4 + 4e][i%4] for e = 0..3.  With lane r pointing at
// S[k0 + r/4][n0 + 4*(r%4)] of a row-major matrix, lane i therefore receives
// S[k0 + e][n0 + i]: four consecutive rows of ONE column -- an MFMA operand
// fragment along the strided dimension, with no transpose in memory.
#pragma once
#include "common.h"

namespace dh {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));

template <typename T> struct Mma;

template <> struct Mma<bf16_t> {
  using Frag = bf16x8;
  static __device__ __forceinline__ floatx16 mma(Frag a, Frag b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mma<f16_t> {
  using Frag = half8;
  static __device__ __forceinline__ floatx16 mma(Frag a, Frag b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// Fragment whose 8 k-values are contiguous in (LDS or global) memory.
template <typename T> __device__ __forceinline__ typename Mma<T>::Frag frag_ld(const T *p) {
  return *reinterpret_cast<const typename Mma<T>::Frag *>(p);
}

// Transposed fragment from row-major LDS `base` (row stride `ld` elements):
// returns S[ka + e][n] for e = 0..3 followed by S[kb + e][n], where n = n0 + (l % 16)
// and the caller passes the lane's own source address pieces:
//   r = l % 16  ->  row offset r / 4, column offset 4 * (r % 4).
template <typename T>
__device__ __forceinline__ typename Mma<T>::Frag frag_ld_tr(const T *base, int ld, int ka, int kb, int n0, int lane) {
  const int r = lane & 15;
  const T *pa = base + (ka + (r >> 2)) * ld + n0 + 4 * (r & 3);
  const T *pb = base + (kb + (r >> 2)) * ld + n0 + 4 * (r & 3);
  typedef short4v __attribute__((address_space(3))) * lds_ptr;
  const short4v a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(pa));
  const short4v b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(pb));
  short8v o;
  o[0] = a[0]; o[1] = a[1]; o[2] = a[2]; o[3] = a[3];
  o[4] = b[0]; o[5] = b[1]; o[6] = b[2]; o[7] = b[3];
  return __builtin_bit_cast(typename Mma<T>::Frag, o);
}

// Pack 8 floats into a 16-bit fragment (round to nearest even).
template <typename T> __device__ __forceinline__ typename Mma<T>::Frag frag_pack(const float *f) {
  typename Mma<T>::Frag o;
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = static_cast<T>(f[j]);
  return o;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---- swizzled 256-byte-row tiles in LDS (head dim 128, 16-bit elements) -------------------------
// A tile is [rows][128] elements with NO padding; the 16-byte chunk index of a row is XORed
// with swz(row), a bijection of row % 16 whose upper two bits enumerate row % 4.  That makes
// both access patterns conflict-free: 16-byte row fragments (16 consecutive rows hit 16
// different chunks) and transpose reads (the 4 rows a half-wave reads land in 4 different
// 64-byte groups).  Tiles are filled by direct global->LDS copies of 1 KB (4 rows) per
// wavefront instruction, the swizzle being applied to the GLOBAL chunk a lane fetches.
__device__ __forceinline__ int swz(int row) { return 4 * (row & 3) + ((row >> 2) & 3); }

// Copy 4 consecutive rows (row0 .. row0+3, each 128 elements) of a row-major global matrix
// into the swizzled tile at `dst4` (wave-uniform LDS address of the 4-row block).  Lane l
// handles row row0 + l/16 and LDS chunk l%16.  `row_g` is the lane's (clamped) global row.
template <typename T>
__device__ __forceinline__ void dma_rows4(const T *gbase, int64_t row_g, int ld, int row_in_tile, int lane, T *dst4) {
  const T *src = gbase + row_g * ld + (((lane & 15) ^ swz(row_in_tile)) * 8);
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                   (__attribute__((address_space(3))) void *)dst4, 16, 0, 0);
}

// 16-byte row fragment (8 consecutive k of one row) from a swizzled tile: row, logical chunk.
template <typename T>
__device__ __forceinline__ typename Mma<T>::Frag frag_ld_swz(const T *tile, int row, int chunk) {
  return frag_ld<T>(tile + row * 128 + ((chunk ^ swz(row)) * 8));
}

// Four transposed fragments (the four 32-column blocks t = 0..3) of a swizzled tile for the
// k rows {ka .. ka+3} u {ka+8 .. ka+11}, ka = k0 + 4*hh, issued as one batch of eight
// transpose reads.  Written in assembly: a builtin would make the compiler wait for every
// direct-to-LDS copy still in flight (it cannot tell the stages apart).  The caller must
// order its uses after tr4_wait<N>().
struct Tr4 { short4v f[8]; };
template <typename T>
__device__ __forceinline__ void tr4_issue(Tr4 &o, const T *tile, int k0, int lane) {
  const int hh = lane >> 5, r = lane & 15;
  const int rowa = k0 + 4 * hh + (r >> 2);
  const int xa = swz(rowa), xb = swz(rowa + 8);
  const uint32_t base = (uint32_t)(uintptr_t)(tile + rowa * 128 + ((r & 3) & 1) * 4);
  const int lc0 = 2 * ((lane >> 4) & 1) + ((r & 3) >> 1);
  uint32_t ad[8];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    ad[2 * t] = base + (((4 * t + lc0) ^ xa) * 16);
    ad[2 * t + 1] = base + 8 * 128 * (uint32_t)sizeof(T) + (((4 * t + lc0) ^ xb) * 16);
  }
  asm volatile("ds_read_b64_tr_b16 %0, %8\n\tds_read_b64_tr_b16 %1, %9\n\t"
               "ds_read_b64_tr_b16 %2, %10\n\tds_read_b64_tr_b16 %3, %11\n\t"
               "ds_read_b64_tr_b16 %4, %12\n\tds_read_b64_tr_b16 %5, %13\n\t"
               "ds_read_b64_tr_b16 %6, %14\n\tds_read_b64_tr_b16 %7, %15"
               : "=&v"(o.f[0]), "=&v"(o.f[1]), "=&v"(o.f[2]), "=&v"(o.f[3]), "=&v"(o.f[4]), "=&v"(o.f[5]),
                 "=&v"(o.f[6]), "=&v"(o.f[7])
               : "v"(ad[0]), "v"(ad[1]), "v"(ad[2]), "v"(ad[3]), "v"(ad[4]), "v"(ad[5]), "v"(ad[6]), "v"(ad[7])
               : "memory");
}
// Wait until at most N LDS reads issued after fragment t of `o` are outstanding, then return fragment t.
// (LDS reads complete in order, so "at most N outstanding" means everything older has landed.)
template <typename T, int N>
__device__ __forceinline__ typename Mma<T>::Frag tr4_get(Tr4 &o, int t) {
  static_assert(N >= 0 && N <= 14 && N % 2 == 0, "even count up to 14");
#define DH_W(n) asm volatile("s_waitcnt lgkmcnt(" #n ")" : "+v"(o.f[2 * t]), "+v"(o.f[2 * t + 1]))
  if (N == 14) DH_W(14); else if (N == 12) DH_W(12); else if (N == 10) DH_W(10); else if (N == 8) DH_W(8);
  else if (N == 6) DH_W(6); else if (N == 4) DH_W(4); else if (N == 2) DH_W(2); else DH_W(0);
#undef DH_W
  short8v o8;
  o8[0] = o.f[2 * t][0]; o8[1] = o.f[2 * t][1]; o8[2] = o.f[2 * t][2]; o8[3] = o.f[2 * t][3];
  o8[4] = o.f[2 * t + 1][0]; o8[5] = o.f[2 * t + 1][1]; o8[6] = o.f[2 * t + 1][2]; o8[7] = o.f[2 * t + 1][3];
  return __builtin_bit_cast(typename Mma<T>::Frag, o8);
}

// ---- LDS reads in assembly ------------------------------------------------------------------------
// The kernels that fill LDS with direct global->LDS copies read it back through these helpers: the
// compiler cannot tell which pipeline stage a read touches and would otherwise wait for every copy in
// flight.  The caller orders each use after lds_wait<N>() on the destination registers (LDS reads
// complete in order: "at most N outstanding" means everything issued earlier has landed).
typedef int int4v __attribute__((ext_vector_type(4)));

// Wait for every global->LDS copy this wavefront has issued (the ones issued in assembly are not
// counted by the compiler).
__device__ __forceinline__ void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <int OFF> __device__ __forceinline__ void lds_read128(int4v &d, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(d) : "v"(addr), "n"(OFF) : "memory");
}
// Eight transpose reads (b64, 16-bit elements) from eight lane addresses plus a common byte offset.
template <int OFF> __device__ __forceinline__ void lds_read_tr8(short4v (&f)[8], const uint32_t (&ad)[8]) {
  asm volatile("ds_read_b64_tr_b16 %0, %8 offset:%16\n\tds_read_b64_tr_b16 %1, %9 offset:%16\n\t"
               "ds_read_b64_tr_b16 %2, %10 offset:%16\n\tds_read_b64_tr_b16 %3, %11 offset:%16\n\t"
               "ds_read_b64_tr_b16 %4, %12 offset:%16\n\tds_read_b64_tr_b16 %5, %13 offset:%16\n\t"
               "ds_read_b64_tr_b16 %6, %14 offset:%16\n\tds_read_b64_tr_b16 %7, %15 offset:%16"
               : "=&v"(f[0]), "=&v"(f[1]), "=&v"(f[2]), "=&v"(f[3]), "=&v"(f[4]), "=&v"(f[5]), "=&v"(f[6]), "=&v"(f[7])
               : "v"(ad[0]), "v"(ad[1]), "v"(ad[2]), "v"(ad[3]), "v"(ad[4]), "v"(ad[5]), "v"(ad[6]), "v"(ad[7]), "n"(OFF)
               : "memory");
}
// Four transpose reads from one lane address plus the byte offsets 0, S, 2 S, 3 S.
template <int S> __device__ __forceinline__ void lds_read_tr4(short4v (&f)[4], uint32_t addr) {
  asm volatile("ds_read_b64_tr_b16 %0, %4\n\tds_read_b64_tr_b16 %1, %4 offset:%5\n\t"
               "ds_read_b64_tr_b16 %2, %4 offset:%6\n\tds_read_b64_tr_b16 %3, %4 offset:%7"
               : "=&v"(f[0]), "=&v"(f[1]), "=&v"(f[2]), "=&v"(f[3])
               : "v"(addr), "n"(S), "n"(2 * S), "n"(3 * S)
               : "memory");
}
template <int N> __device__ __forceinline__ void lds_wait(int4v &d) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(d) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait(int4v &a, int4v &b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait(short4v &a, short4v &b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait(short4v &a, short4v &b, short4v &c, short4v &d) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
}
template <typename T> __device__ __forceinline__ typename Mma<T>::Frag frag_join(const short4v &a, const short4v &b) {
  short8v o8;
  o8[0] = a[0]; o8[1] = a[1]; o8[2] = a[2]; o8[3] = a[3];
  o8[4] = b[0]; o8[5] = b[1]; o8[6] = b[2]; o8[7] = b[3];
  return __builtin_bit_cast(typename Mma<T>::Frag, o8);
}

// ---- global -> LDS tile copies of the d = 128 attention kernels ----------------------------------
// Per-lane constants of the general (clamped) K/V tile copies.
struct CopyLane {
  int lrow, l16;         // row inside a 4-row copy block, 16-byte chunk slot
};

// One 1 KB copy (4 rows of a K or V tile) in its fast form: wave-uniform 64-bit global base, the lane's
// 32-bit byte offset, wave-uniform LDS byte address.  The compiler does not count these copies: the
// kernel waits for them itself (dma_wait_all) before the barrier that publishes a stage.
__device__ __forceinline__ void dma_block_fast(const char *base, uint32_t lane_off, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_off), "s"(base), "s"(lds_dst)
               : "memory", "m0");
}

// NBLK copy blocks (4 rows each, consecutive rows of one tile) of a wavefront in general form: rows past the last key
// are clamped per lane (they are masked in the scores, and their V rows meet zero probabilities).  Kept
// as a rolled loop: it runs once per query tile and for tiles that reach past the keys.
// `swz_v`: the tile uses swz(row) (transpose-read tiles) instead of row % 16 (row-fragment tiles).
template <typename T, int NBLK = 8>
__device__ __forceinline__ void dma_tile32_general(T *dst, const T *g, int stride, int swz_v, int row0_g, int row0_t, int sk,
                                                  const CopyLane &cl) {
  asm volatile("" : "+s"(row0_g));               // keep the address arithmetic next to the copies
#pragma unroll 1
  for (int i = 0; i < NBLK; ++i) {
    int kr = row0_g + 4 * i + cl.lrow;
    kr = kr < sk ? kr : sk - 1;
    const int row = row0_t + 4 * i + cl.lrow;
    const int f = swz_v ? (4 * (row & 3) + ((row >> 2) & 3)) : (row & 15);
    const T *src = g + (int64_t)kr * stride + ((cl.l16 ^ f) * 8);
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                     (__attribute__((address_space(3))) void *)(dst + i * 512), 16, 0, 0);
  }
}

// Reductions over the lane pair (l, l ^ 32) with v_permlane32_swap (VALU) instead of a shuffle through the
// LDS crossbar: swapping the upper half of one copy of x with the lower half of another leaves, in every
// lane, its own value in one result and its partner's in the other.
__device__ __forceinline__ float pair32_max(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair32_sum(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Row index inside a 32-row accumulator block held by register v of lane half h.
__device__ __forceinline__ int acc_row(int v, int h) { return 8 * (v >> 2) + 4 * h + (v & 3); }

// Workgroups reach the 8 XCDs round-robin by linear id and each XCD has its own L2.  Split a linear id over
// G groups of I items so that the workgroups of one group (which re-read the same rows) stay on as few XCDs
// as possible: whole groups per XCD when G divides by 8, one group per 8 / G XCDs when G divides 8.
__device__ __forceinline__ void xcd_group_item(int id, int G, int I, int &g, int &i) {
  const int x = id & 7, n = id >> 3;
  if ((G & 7) == 0) {
    g = x + 8 * (n / I);
    i = n % I;
  } else if (8 % G == 0 && ((G * I) & 7) == 0) {
    g = x % G;
    i = x / G + (8 / G) * n;
  } else {
    g = id % G;
    i = id / G;
  }
}

}  // namespace dh

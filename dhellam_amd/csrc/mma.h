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

// Row index inside a 32-row accumulator block held by register v of lane half h.
__device__ __forceinline__ int acc_row(int v, int h) { return 8 * (v >> 2) + 4 * h + (v & 3); }

}  // namespace dh

// out[c][r] = in[r][c] for 16-bit elements, through LDS transpose reads.
//
// Used in front of the weight-gradient GEMM: dW = dY^T X reads both operands along their strided
// dimension, the slowest layout for the GEMM library on this machine (measured 1.0 PFLOP/s at the
// 70B-shard shapes against 1.2 with dY^T materialised row-major), and a transpose at HBM speed costs
// less than that difference once the other operand is a few thousand columns wide.
//
// A workgroup moves a [64 rows][256 cols] tile: coalesced 16-byte loads, LDS rows padded to 544 bytes
// (the four rows a 16-lane group reads land in different banks), then every lane gathers 8 consecutive
// rows of ONE column with two ds_read_b64_tr_b16 and stores them as 16 contiguous bytes of the output
// row; a lane writes a full 128-byte line of its output row over the 8 steps.
#include "mma.h"

namespace dh {

template <bool NT>
__global__ void __launch_bounds__(256) transpose16_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                                          int64_t rows, int64_t cols, int64_t ld_in, int64_t ld_out) {
  constexpr int TR = 64, TC = 256, PITCH = TC * 2 + 32;       // bytes
  __shared__ __attribute__((aligned(16))) unsigned char tile[TR * PITCH];
  const int64_t r0 = (int64_t)blockIdx.y * TR, c0 = (int64_t)blockIdx.x * TC;
  const int tid = threadIdx.x;
  // load: thread t -> row t / 32 + 8 i, 16-byte chunk t % 32
  {
    const int lr = tid >> 5, ch = tid & 31;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = lr + 8 * i;
      Vec<uint16_t> v;
#pragma unroll
      for (int j = 0; j < 8; ++j) v.v[j] = 0;
      if (r0 + r < rows && c0 + ch * 8 < cols) v = ldg_s<NT>(in + (r0 + r) * ld_in + c0 + ch * 8);
      *reinterpret_cast<Vec<uint16_t> *>(tile + r * PITCH + ch * 16) = v;
    }
  }
  __syncthreads();
  // transpose reads: lane l of wave w owns column 64 w + 16 (l / 16) + l % 16 of the tile; a read with the lane
  // address &tile[k0 + r / 4][n0 + 4 (r % 4)] (r = l % 16, n0 = the group's first column) returns rows k0..k0+3
  // of the lane's column.
  const int lane = tid & 63, w = tid >> 6;
  const int r = lane & 15, n0 = 64 * w + 16 * (lane >> 4);
  const int col = n0 + r;
  typedef short4v __attribute__((address_space(3))) *lds_tr;
  const uint32_t base = (uint32_t)(uintptr_t)tile + (uint32_t)((r >> 2) * PITCH + (n0 + 4 * (r & 3)) * 2);
  // Every lane takes part in the reads (a lane's result comes from the addresses its neighbours supply);
  // only the stores are guarded.
  const bool col_ok = c0 + col < cols;
  uint16_t *orow = out + (c0 + col) * ld_out + r0;
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const short4v a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(base + (uint32_t)((8 * s) * PITCH)));
    const short4v b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(base + (uint32_t)((8 * s + 4) * PITCH)));
    if (col_ok && r0 + 8 * s < rows) {        // rows are a multiple of 8: a step is all in or all out
      Vec<uint16_t> o;
      o.v[0] = (uint16_t)a[0]; o.v[1] = (uint16_t)a[1]; o.v[2] = (uint16_t)a[2]; o.v[3] = (uint16_t)a[3];
      o.v[4] = (uint16_t)b[0]; o.v[5] = (uint16_t)b[1]; o.v[6] = (uint16_t)b[2]; o.v[7] = (uint16_t)b[3];
      stg_s<NT>(orow + 8 * s, o);
    }
  }
}

}  // namespace dh

extern "C" int dh_transpose_2d(const void *in, void *out, int64_t rows, int64_t cols, int64_t ld_in, int64_t ld_out,
                               int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(rows >= 0 && cols >= 0, "negative size");
  if (rows == 0 || cols == 0) return DH_OK;
  DH_CHECK(in && out, "null pointer");
  DH_CHECK(dtype == DH_BF16 || dtype == DH_F16, "transpose supports 16-bit element types (dtype %d)", dtype);
  DH_CHECK(rows % 8 == 0 && cols % 8 == 0 && ld_in % 8 == 0 && ld_out % 8 == 0 && ld_in >= cols && ld_out >= rows,
           "rows=%lld cols=%lld ld_in=%lld ld_out=%lld: sizes and leading dimensions must be multiples of 8",
           (long long)rows, (long long)cols, (long long)ld_in, (long long)ld_out);
  DH_CHECK(aligned16(in) && aligned16(out), "in/out must be 16-byte aligned");
  const dim3 grid((unsigned)cdiv(cols, 256), (unsigned)cdiv(rows, 64));
  DH_CHECK(grid.y < 65536, "too many rows for one launch");
  if (stream_hint(4 * rows * cols))
    hipLaunchKernelGGL(transpose16_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)in,
                       (uint16_t *)out, rows, cols, ld_in, ld_out);
  else
    hipLaunchKernelGGL(transpose16_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)in,
                       (uint16_t *)out, rows, cols, ld_in, ld_out);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

// out[c][r] = in[r][c] for 16-bit elements, staged through LDS.
//
// Used in front of the weight-gradient GEMM: dW = dY^T X reads both operands along their strided
// dimension, the slowest layout for the GEMM library on this machine (measured 1.0 PFLOP/s at the
// 70B-shard shapes against 1.2 with dY^T materialised row-major), and a transpose at HBM speed costs
// less than that difference once the other operand is a few thousand columns wide.
//
// A workgroup moves a [64 rows][256 cols] tile: coalesced 16-byte loads into LDS rows of 129 dwords,
// then every lane gathers 8 consecutive rows of ONE column (two-byte LDS reads, conflict-free: 8-row
// steps land 8 banks apart) and stores them as 16 contiguous bytes of the output row.  The 8 lanes that
// share a column are adjacent, so one store instruction writes 8 whole 128-byte lines.  A first version
// built the same 16 bytes with LDS transpose reads, which tie adjacent lanes to adjacent COLUMNS: its
// store instructions touched 64 lines with 16 bytes each and ran at 3.8 TB/s where this one reaches 5.6-6.2
// ([4096 x 8192] in 24 us instead of 35).
#include "mma.h"

namespace dh {

__global__ void __launch_bounds__(256) transpose16_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                                          int64_t rows, int64_t cols, int64_t ld_in, int64_t ld_out) {
  constexpr int TR = 64, TC = 256, PITCH = TC * 2 + 4;       // bytes; 129 dwords: 8-row steps land 8 banks apart
  __shared__ __attribute__((aligned(16))) unsigned char tile[TR * PITCH];
  const int64_t r0 = (int64_t)blockIdx.y * TR, c0 = (int64_t)blockIdx.x * TC;
  const int tid = threadIdx.x;
  {
    const int lr = tid >> 5, ch = tid & 31;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = lr + 8 * i;
      dh_u32x4 v = {0, 0, 0, 0};
      if (r0 + r < rows && c0 + ch * 8 < cols)
        v = *reinterpret_cast<const dh_u32x4 *>(in + (r0 + r) * ld_in + c0 + ch * 8);
      uint32_t *d = reinterpret_cast<uint32_t *>(tile + r * PITCH + ch * 16);
      d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
    }
  }
  __syncthreads();
  const int lane = tid & 63, w = tid >> 6;
  const int rb = lane & 7, cl = lane >> 3;                    // 8-row block, column within the step
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const int col = 64 * w + 8 * s + cl;
    const unsigned char *src = tile + (8 * rb) * PITCH + col * 2;
    Vec<uint16_t> o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o.v[j] = *reinterpret_cast<const uint16_t *>(src + j * PITCH);
    if (c0 + col < cols && r0 + 8 * rb < rows) stg_s<false>(out + (c0 + col) * ld_out + r0 + 8 * rb, o);
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
  {
    const char *a = (const char *)in, *b = (const char *)out;
    const int64_t na = (rows - 1) * ld_in * 2 + cols * 2, nb = (cols - 1) * ld_out * 2 + rows * 2;
    DH_CHECK(a + na <= b || b + nb <= a, "in and out overlap: the transpose is not in place");
  }
  const dim3 grid((unsigned)cdiv(cols, 256), (unsigned)cdiv(rows, 64));
  DH_CHECK(grid.y < 65536, "too many rows for one launch");
  // Plain (cached) accesses at every size: non-temporal ones measured 5-25 % slower here.
  hipLaunchKernelGGL(transpose16_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)in, (uint16_t *)out,
                     rows, cols, ld_in, ld_out);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

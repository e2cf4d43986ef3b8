// Single-pass merge of ring-attention partial results.
//
// For query row t and head h, over the steps s that produced a partial for that
// row:  lse = logsumexp_s(lse_s),  out = sum_s out_s * exp(lse_s - lse).
// One lane owns one 16-byte chunk of one (row, head); the few lse values are
// re-read per chunk (they are 1/64th of the traffic).  Everything is fp32 with a
// running-max logsumexp; partial outputs are read exactly once.
#include "common.h"

namespace dh {

constexpr int MERGE_MAX_STEPS = 8;

struct MergeParams {
  const void *outs[MERGE_MAX_STEPS];
  const float *lses[MERGE_MAX_STEPS];
  int row_begin[MERGE_MAX_STEPS];
  int rows[MERGE_MAX_STEPS];
  int n_steps;
  void *out;
  float *lse;
  int batch, sq, hq, d;
};

// exp(x) for x <= 0 and log(x) for x >= 1 through the hardware's base-2 instructions (1 ulp): a lane evaluates
// 2 n_steps exponentials per 16-byte chunk, and with the library routines those instructions outnumbered the
// memory instructions twenty to one.
__device__ __forceinline__ float exp_neg(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float log_pos(float x) { return __builtin_amdgcn_logf(x) * 0.6931471805599453f; }

// IDX: the type the item index is taken apart in (three divisions by run-time sizes stand in front of an item's
// loads: 32-bit ones whenever the item count allows).
template <typename T, int NS, typename IDX>
__global__ void __launch_bounds__(256) attn_merge_kernel(const MergeParams p) {
  constexpr int N = Vec<T>::N;
  const IDX cpr = (IDX)(p.d / N);  // chunks per (row, head)
  const IDX nitems = (IDX)p.batch * (IDX)p.sq * (IDX)p.hq * cpr;
  const IDX hq_ = (IDX)p.hq, sq_ = (IDX)p.sq;
  for (IDX it = (IDX)blockIdx.x * 256 + threadIdx.x; it < nitems; it += (IDX)gridDim.x * 256) {
    const int ch = (int)(it % cpr);
    IDX r = it / cpr;
    const int h = (int)(r % hq_);
    r /= hq_;
    const int t = (int)(r % sq_);
    const int b = (int)(r / sq_);
    // every load of the item goes out before any arithmetic: the partial outputs do not depend on the weights
    float ls[NS];
    Vec<T> x[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      ls[s] = -INFINITY;
      const int rr = t - p.row_begin[s];
      if (rr >= 0 && rr < p.rows[s]) {
        ls[s] = p.lses[s][((int64_t)b * p.hq + h) * p.rows[s] + rr];
        x[s] = ldg(reinterpret_cast<const T *>(p.outs[s]) + (((int64_t)b * p.rows[s] + rr) * p.hq + h) * p.d + ch * N);
      }
    }
    float m = -INFINITY;
#pragma unroll
    for (int s = 0; s < NS; ++s) m = fmaxf(m, ls[s]);
    float sum = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s)
      if (ls[s] > -INFINITY) sum += exp_neg(ls[s] - m);
    const float lse = sum > 0.f ? m + log_pos(sum) : -INFINITY;
    float acc[N];
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      if (ls[s] > -INFINITY) {
        const float w = exp_neg(ls[s] - lse);
#pragma unroll
        for (int j = 0; j < N; ++j) acc[j] += w * to_f(x[s].v[j]);
      }
    }
    Vec<T> o;
#pragma unroll
    for (int j = 0; j < N; ++j) o.v[j] = from_f<T>(acc[j]);
    stg(reinterpret_cast<T *>(p.out) + (((int64_t)b * p.sq + t) * p.hq + h) * p.d + ch * N, o);
    if (ch == 0) p.lse[((int64_t)b * p.hq + h) * p.sq + t] = lse;
  }
}

}  // namespace dh

extern "C" int dh_attn_merge(const void *const *outs, const float *const *lses, const int32_t *row_begin,
                             const int32_t *rows, int n_steps, void *out, float *lse, int batch, int sq, int hq,
                             int d, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(n_steps >= 1 && n_steps <= MERGE_MAX_STEPS, "n_steps=%d must be in [1, %d]", n_steps, MERGE_MAX_STEPS);
  DH_CHECK(batch >= 0 && sq >= 0 && hq > 0 && d > 0, "bad shape");
  if (batch == 0 || sq == 0) return DH_OK;
  DH_CHECK(outs && lses && row_begin && rows && out && lse, "null pointer");
  const int n = 16 / (int)dtype_size(dtype);
  DH_CHECK(d % n == 0, "head dim %d must be a multiple of %d", d, n);
  MergeParams p;
  for (int s = 0; s < MERGE_MAX_STEPS; ++s) {
    p.outs[s] = nullptr; p.lses[s] = nullptr; p.row_begin[s] = 0; p.rows[s] = 0;
  }
  for (int s = 0; s < n_steps; ++s) {
    DH_CHECK(outs[s] && lses[s], "null partial at step %d", s);
    DH_CHECK(aligned16(outs[s]), "partial output %d must be 16-byte aligned", s);
    DH_CHECK(row_begin[s] >= 0 && rows[s] >= 0 && row_begin[s] + rows[s] <= sq,
             "step %d covers rows [%d, %d) outside [0, %d)", s, row_begin[s], row_begin[s] + rows[s], sq);
    p.outs[s] = outs[s]; p.lses[s] = lses[s]; p.row_begin[s] = row_begin[s]; p.rows[s] = rows[s];
  }
  DH_CHECK(aligned16(out), "out must be 16-byte aligned");
  p.n_steps = n_steps; p.out = out; p.lse = lse; p.batch = batch; p.sq = sq; p.hq = hq; p.d = d;
  const int64_t nitems = (int64_t)batch * sq * hq * (d / n);
  int64_t blocks = cdiv(nitems, 256);
  if (blocks > 256 * 32) blocks = 256 * 32;
  // steps beyond n_steps cover no rows (rows = 0), so a kernel compiled for more steps than given skips them
  const bool small = nitems + blocks * 256 < (1ll << 32);
#define DH_MERGE(NS)                                                                                                   \
  do {                                                                                                                 \
    if (small) hipLaunchKernelGGL((attn_merge_kernel<T, NS, uint32_t>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, p); \
    else hipLaunchKernelGGL((attn_merge_kernel<T, NS, int64_t>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, p);        \
  } while (0)
  DH_DISPATCH_DTYPE(dtype, {
    if (n_steps <= 2) DH_MERGE(2); else if (n_steps <= 4) DH_MERGE(4); else DH_MERGE(8);
  });
#undef DH_MERGE
  DH_LAUNCH_CHECK();
  return DH_OK;
}

// MoE routing and token permutation for one expert-parallel rank.
//
// Index work is exact integer arithmetic:
//   route : top-k of the logits per token (descending value, ties to the lower
//           expert id), gates = softmax over the k selected logits.
//   sort  : STABLE counting sort of the flat assignment list (token-major,
//           assignment a = token*k + j) by expert id: per-block histogram ->
//           exclusive scan over (expert, block) -> ranked scatter.  Stability
//           comes from ranking with wave ballots in item order, not from atomics.
// Row movement is HBM-bound: one workgroup per row, 16-byte accesses.
//   gather  : permuted[r] = scale * x[token of the r-th sorted local assignment]
//   scatter : out[t] = sum_j gate * y[row of (t, j)]   (fixed j order, fp32)
// Row counts live on the device (expert_offsets), so nothing here syncs the host.
#include "common.h"
#include <mutex>

namespace dh {

constexpr int MOE_MAX_E = 64;
constexpr int MOE_MAX_K = 8;
constexpr int SORT_ITEMS = 1024;  // assignments per block (4 rounds of 256)

__global__ void __launch_bounds__(256)
moe_route_kernel(const float *__restrict__ logits, int32_t *__restrict__ topk_idx, float *__restrict__ gates,
                 int64_t tokens, int E, int K) {
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < tokens; t += (int64_t)gridDim.x * 256) {
    const float *row = logits + t * E;
    uint64_t taken = 0;
    float sel[MOE_MAX_K];
    int idx[MOE_MAX_K];
#pragma unroll
    for (int j = 0; j < MOE_MAX_K; ++j) {
      if (j < K) {
        int best = -1;
        float bv = 0.f;
        for (int e = 0; e < E; ++e) {
          if ((taken >> e) & 1) continue;
          const float v = row[e];
          // strict > keeps the lowest expert id among equal values; NaN never wins
          if (best < 0 || v > bv) {
            best = e;
            bv = v;
          }
        }
        taken |= (uint64_t)1 << best;
        sel[j] = bv;
        idx[j] = best;
      }
    }
    float den = 0.f;
    float ex[MOE_MAX_K];
#pragma unroll
    for (int j = 0; j < MOE_MAX_K; ++j)
      if (j < K) {
        ex[j] = expf(sel[j] - sel[0]);
        den += ex[j];
      }
#pragma unroll
    for (int j = 0; j < MOE_MAX_K; ++j)
      if (j < K) {
        topk_idx[t * K + j] = idx[j];
        gates[t * K + j] = ex[j] / den;
      }
  }
}

// hist [nblocks][E]
__global__ void __launch_bounds__(256)
moe_hist_kernel(const int32_t *__restrict__ expert_of, int32_t *__restrict__ hist, int64_t n, int E) {
  __shared__ int cnt[MOE_MAX_E];
  if (threadIdx.x < MOE_MAX_E) cnt[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * SORT_ITEMS;
#pragma unroll
  for (int r = 0; r < SORT_ITEMS / 256; ++r) {
    const int64_t i = base + r * 256 + threadIdx.x;
    if (i < n) {
      const int e = expert_of[i];
      if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);  // ids outside [0, E) are left out of the sort
    }
  }
  __syncthreads();
  if ((int)threadIdx.x < E) hist[(int64_t)blockIdx.x * E + threadIdx.x] = cnt[threadIdx.x];
}

// One block: per expert, exclusive scan of its per-block counts; expert bases from totals.
// hist is overwritten with the starting position of (block, expert) in the sorted order.
__global__ void __launch_bounds__(64)
moe_scan_kernel(int32_t *__restrict__ hist, int32_t *__restrict__ tokens_per_expert,
                int32_t *__restrict__ expert_offsets, int nblocks, int E) {
  __shared__ int total[MOE_MAX_E], base[MOE_MAX_E + 1];
  const int e = threadIdx.x;
  if (e < E) {
    int run = 0;
    for (int b = 0; b < nblocks; ++b) {
      const int c = hist[(int64_t)b * E + e];
      hist[(int64_t)b * E + e] = run;
      run += c;
    }
    total[e] = run;
    tokens_per_expert[e] = run;
  }
  __syncthreads();
  if (e == 0) {
    int run = 0;
    for (int i = 0; i < E; ++i) {
      base[i] = run;
      run += total[i];
    }
    base[E] = run;
    for (int i = 0; i <= E; ++i) expert_offsets[i] = base[i];
  }
  __syncthreads();
  if (e < E) {
    const int bs = base[e];
    for (int b = 0; b < nblocks; ++b) hist[(int64_t)b * E + e] += bs;
  }
}

__global__ void __launch_bounds__(256)
moe_rank_scatter_kernel(const int32_t *__restrict__ expert_of, const int32_t *__restrict__ start,
                        int32_t *__restrict__ sorted_idx, int32_t *__restrict__ dest_row, int64_t n, int E) {
  __shared__ int running[MOE_MAX_E];
  __shared__ int wcnt[4][MOE_MAX_E];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if ((int)threadIdx.x < E) running[threadIdx.x] = start[(int64_t)blockIdx.x * E + threadIdx.x];
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * SORT_ITEMS;
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  for (int r = 0; r < SORT_ITEMS / 256; ++r) {
    const int64_t i = base + r * 256 + threadIdx.x;
    int my = i < n ? expert_of[i] : -1;
    if (my >= E) my = -1;  // an id outside [0, E) gets no place (its dest_row is -1)
    int rank_in_wave = 0;
    for (int e = 0; e < E; ++e) {
      const uint64_t m = __ballot(my == e);
      if (lane == 0) wcnt[w][e] = __popcll(m);
      if (my == e) rank_in_wave = __popcll(m & lt_mask);
    }
    __syncthreads();
    if (my >= 0) {
      int pos = running[my] + rank_in_wave;
      for (int ww = 0; ww < w; ++ww) pos += wcnt[ww][my];
      dest_row[i] = pos;
      sorted_idx[pos] = (int32_t)i;
    } else if (i < n) {
      dest_row[i] = -1;
    }
    __syncthreads();
    if ((int)threadIdx.x < E) running[threadIdx.x] += wcnt[0][threadIdx.x] + wcnt[1][threadIdx.x] + wcnt[2][threadIdx.x] + wcnt[3][threadIdx.x];
    __syncthreads();
  }
}

// A workgroup moves RPB rows per trip and issues every load of the trip before its first store: a row is only
// hidden / N / 256 (2 at hidden 4096) vectors per lane, and one row per workgroup left the copy latency-bound.
// Rows past max_rows are never written, whatever expert_offsets says (the caller sized `permuted` by it).
template <typename T, int RPB>
__global__ void __launch_bounds__(256)
moe_gather_kernel(const T *__restrict__ x, const int32_t *__restrict__ sorted_idx, const float *__restrict__ row_scale,
                  T *__restrict__ permuted, const int32_t *__restrict__ offs, int e_lo, int e_hi, int64_t max_rows,
                  int K, int64_t hidden, int vec_ok) {
  constexpr int N = Vec<T>::N;
  constexpr int U = 2;
  const int first = offs[e_lo];
  int64_t n_rows = (int64_t)offs[e_hi] - first;
  if (n_rows > max_rows) n_rows = max_rows;
  if (n_rows < 0) n_rows = 0;
  // rows between the real count and max_rows are zeroed, so the caller may hand over uninitialised memory
  for (int64_t r = n_rows + blockIdx.x; r < max_rows; r += gridDim.x) {
    T *dst = permuted + r * hidden;
    if (vec_ok) {
      Vec<T> z;
#pragma unroll
      for (int j = 0; j < N; ++j) z.v[j] = from_f<T>(0.f);
      for (int64_t c = threadIdx.x; c < hidden / N; c += 256) stg(dst + c * N, z);
    } else {
      for (int64_t c = threadIdx.x; c < hidden; c += 256) dst[c] = from_f<T>(0.f);
    }
  }
  for (int64_t r0 = (int64_t)blockIdx.x * RPB; r0 < n_rows; r0 += (int64_t)gridDim.x * RPB) {
    const T *src[RPB];
    float sc[RPB];
#pragma unroll
    for (int i = 0; i < RPB; ++i) {
      const int64_t r = r0 + i < n_rows ? r0 + i : n_rows - 1;
      const int a = sorted_idx[first + r];
      src[i] = x + (int64_t)(a / K) * hidden;
      sc[i] = row_scale ? row_scale[a] : 1.0f;
    }
    if (vec_ok) {
      const int64_t nv = hidden / N;
      for (int64_t c0 = threadIdx.x; c0 < nv; c0 += U * 256) {
        Vec<T> v[RPB][U];
#pragma unroll
        for (int i = 0; i < RPB; ++i)
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (c0 + u * 256 < nv) v[i][u] = ldg(src[i] + (c0 + u * 256) * N);
#pragma unroll
        for (int i = 0; i < RPB; ++i) {
          if (r0 + i < n_rows) {
            T *dst = permuted + (r0 + i) * hidden;
#pragma unroll
            for (int u = 0; u < U; ++u) {
              if (c0 + u * 256 < nv) {
                if (row_scale) {
#pragma unroll
                  for (int j = 0; j < N; ++j) v[i][u].v[j] = from_f<T>(to_f(v[i][u].v[j]) * sc[i]);
                }
                stg(dst + (c0 + u * 256) * N, v[i][u]);
              }
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < RPB; ++i) {
        if (r0 + i < n_rows) {
          T *dst = permuted + (r0 + i) * hidden;
          for (int64_t c = threadIdx.x; c < hidden; c += 256)
            dst[c] = row_scale ? from_f<T>(to_f(src[i][c]) * sc[i]) : src[i][c];
        }
      }
    }
  }
}

// A workgroup combines TPB tokens per trip; all row loads of the trip are issued before the first store.
// KT: compile-time bound of the slots per token (K <= KT), so the slot loops unroll to what is needed.
template <typename T, int TPB, int KT>
__global__ void __launch_bounds__(256)
moe_scatter_kernel(const T *__restrict__ y, const int32_t *__restrict__ dest_row, const float *__restrict__ gates,
                   T *__restrict__ out, const int32_t *__restrict__ offs, int e_lo, int e_hi, int64_t tokens, int K,
                   int64_t hidden, int vec_ok) {
  constexpr int N = Vec<T>::N;
  const int first = offs[e_lo];
  const int64_t n_rows = (int64_t)offs[e_hi] - first;
  for (int64_t t0 = (int64_t)blockIdx.x * TPB; t0 < tokens; t0 += (int64_t)gridDim.x * TPB) {
    int rows[TPB][KT];
    float wts[TPB][KT];
#pragma unroll
    for (int i = 0; i < TPB; ++i)
#pragma unroll
      for (int j = 0; j < KT; ++j) {
        rows[i][j] = -1;
        wts[i][j] = 0.f;
        if (j < K && t0 + i < tokens) {
          const int64_t rr = (int64_t)dest_row[(t0 + i) * K + j] - first;
          if (rr >= 0 && rr < n_rows) {
            rows[i][j] = (int)rr;
            wts[i][j] = gates ? gates[(t0 + i) * K + j] : 1.0f;
          }
        }
      }
    if (vec_ok) {
      for (int64_t c = threadIdx.x; c < hidden / N; c += 256) {
        Vec<T> v[TPB][KT];
#pragma unroll
        for (int i = 0; i < TPB; ++i)
#pragma unroll
          for (int j = 0; j < KT; ++j)
            if (rows[i][j] >= 0) v[i][j] = ldg(y + (int64_t)rows[i][j] * hidden + c * N);
#pragma unroll
        for (int i = 0; i < TPB; ++i) {
          if (t0 + i < tokens) {
            float acc[N];
#pragma unroll
            for (int e = 0; e < N; ++e) acc[e] = 0.f;
#pragma unroll
            for (int j = 0; j < KT; ++j)
              if (rows[i][j] >= 0) {
#pragma unroll
                for (int e = 0; e < N; ++e) acc[e] += wts[i][j] * to_f(v[i][j].v[e]);
              }
            Vec<T> o;
#pragma unroll
            for (int e = 0; e < N; ++e) o.v[e] = from_f<T>(acc[e]);
            stg(out + (t0 + i) * hidden + c * N, o);
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < TPB; ++i) {
        if (t0 + i < tokens) {
          for (int64_t c = threadIdx.x; c < hidden; c += 256) {
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < KT; ++j)
              if (rows[i][j] >= 0) acc += wts[i][j] * to_f(y[(int64_t)rows[i][j] * hidden + c]);
            out[(t0 + i) * hidden + c] = from_f<T>(acc);
          }
        }
      }
    }
  }
}

// dgates[t*K + j] = <dout[t], y[row(t, j)]>, 0 for assignments that are not local.
template <typename T>
__global__ void __launch_bounds__(256)
moe_gate_grad_kernel(const T *__restrict__ dout, const T *__restrict__ y, const int32_t *__restrict__ dest_row,
                     float *__restrict__ dgates, const int32_t *__restrict__ offs, int e_lo, int e_hi, int64_t tokens,
                     int K, int64_t hidden, int vec_ok) {
  __shared__ float red[4];
  const int first = offs[e_lo], n_rows = offs[e_hi] - first;
  for (int64_t a = blockIdx.x; a < tokens * K; a += gridDim.x) {
    const int rr = dest_row[a] - first;
    float s = 0.f;
    if (rr >= 0 && rr < n_rows) {  // uniform over the block
      const T *p = dout + (a / K) * hidden;
      const T *q = y + (int64_t)rr * hidden;
      if (vec_ok) {
        constexpr int N = Vec<T>::N;
        for (int64_t c = threadIdx.x; c < hidden / N; c += 256) {
          const Vec<T> pv = ldg(p + c * N), qv = ldg(q + c * N);
#pragma unroll
          for (int e = 0; e < N; ++e) s += to_f(pv.v[e]) * to_f(qv.v[e]);
        }
      } else {
        for (int64_t c = threadIdx.x; c < hidden; c += 256) s += to_f(p[c]) * to_f(q[c]);
      }
    }
    s = block256_sum(s, red);
    if (threadIdx.x == 0) dgates[a] = s;
  }
}

}  // namespace dh

extern "C" int dh_moe_route_topk(const float *logits, int32_t *topk_idx, float *gates, int64_t tokens, int experts,
                                 int k, void *stream) {
  using namespace dh;
  DH_CHECK(tokens >= 0, "tokens must be >= 0");
  DH_CHECK(experts >= 1 && experts <= MOE_MAX_E, "experts=%d must be in [1, %d]", experts, MOE_MAX_E);
  DH_CHECK(k >= 1 && k <= MOE_MAX_K && k <= experts, "k=%d must be in [1, min(%d, experts)]", k, MOE_MAX_K);
  if (tokens == 0) return DH_OK;
  DH_CHECK(logits && topk_idx && gates, "null pointer");
  int64_t blocks = cdiv(tokens, 256);
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, logits, topk_idx,
                     gates, tokens, experts, k);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" size_t dh_moe_sort_workspace_bytes(int64_t n_assign, int experts) {
  const int64_t nb = n_assign > 0 ? dh::cdiv(n_assign, dh::SORT_ITEMS) : 1;
  return (size_t)(nb * (experts > 0 ? experts : 1) * sizeof(int32_t)) + 16;
}

static int moe_sort_launch(const int32_t *topk_idx, int32_t *tokens_per_expert, int32_t *expert_offsets,
                           int32_t *sorted_idx, int32_t *dest_row, int32_t *hist, int64_t n_assign, int experts,
                           hipStream_t st) {
  using namespace dh;
  const int nb = (int)cdiv(n_assign, SORT_ITEMS);
  if (nb > 0) {
    DH_CHECK(topk_idx && sorted_idx && dest_row, "null pointer");
    hipLaunchKernelGGL(moe_hist_kernel, dim3(nb), dim3(256), 0, st, topk_idx, hist, n_assign, experts);
  }
  hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(64), 0, st, hist, tokens_per_expert, expert_offsets, nb, experts);
  if (nb > 0)
    hipLaunchKernelGGL(moe_rank_scatter_kernel, dim3(nb), dim3(256), 0, st, topk_idx, hist, sorted_idx, dest_row,
                       n_assign, experts);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_moe_sort(const int32_t *topk_idx, int32_t *tokens_per_expert, int32_t *expert_offsets,
                           int32_t *sorted_idx, int32_t *dest_row, void *workspace, size_t workspace_bytes,
                           int64_t n_assign, int experts, void *stream) {
  using namespace dh;
  DH_CHECK(n_assign >= 0 && n_assign < (1ll << 31), "n_assign out of range");
  DH_CHECK(experts >= 1 && experts <= MOE_MAX_E, "experts=%d must be in [1, %d]", experts, MOE_MAX_E);
  DH_CHECK(tokens_per_expert && expert_offsets && workspace, "null pointer");
  DH_CHECK(workspace_bytes >= dh_moe_sort_workspace_bytes(n_assign, experts),
           "workspace of %zu bytes is smaller than dh_moe_sort_workspace_bytes(%lld, %d) = %zu", workspace_bytes,
           (long long)n_assign, experts, dh_moe_sort_workspace_bytes(n_assign, experts));
  return moe_sort_launch(topk_idx, tokens_per_expert, expert_offsets, sorted_idx, dest_row, (int32_t *)workspace,
                         n_assign, experts, (hipStream_t)stream);
}

// ---- the sort for callers that cannot allocate ---------------------------------------------------------------
// The per-block histogram / start-position table lives in a file-scope device array instead of a caller's
// workspace.  The array's name is only a host-side handle: its device address is asked for once per device
// (hipGetSymbolAddress, with that device current) and every launch gets that address.
constexpr int64_t MOE_STATIC_MAX_ASSIGN = 1ll << 20;
constexpr int MOE_STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) int32_t scratch[(MOE_STATIC_MAX_ASSIGN / dh::SORT_ITEMS) * dh::MOE_MAX_E];
static int32_t *g_scratch_ptr[MOE_STATIC_MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int moe_static_scratch(int32_t **out) {
  int dev = -1;
  DH_HIP(hipGetDevice(&dev));
  DH_CHECK(dev >= 0 && dev < MOE_STATIC_MAX_DEVICES, "device %d outside [0, %d)", dev, MOE_STATIC_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    DH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    DH_CHECK(p != nullptr, "no device address for the static sort table");
    g_scratch_ptr[dev] = (int32_t *)p;
  }
  *out = g_scratch_ptr[dev];
  return DH_OK;
}

extern "C" int64_t dh_moe_sort_static_max_assign(void) { return MOE_STATIC_MAX_ASSIGN; }

extern "C" int dh_moe_sort_static(const int32_t *topk_idx, int32_t *tokens_per_expert, int32_t *expert_offsets,
                                  int32_t *sorted_idx, int32_t *dest_row, int64_t n_assign, int experts,
                                  void *stream) {
  using namespace dh;
  DH_CHECK(n_assign >= 0 && n_assign <= MOE_STATIC_MAX_ASSIGN,
           "n_assign=%lld exceeds what the static table holds (%lld); use dh_moe_sort with a workspace",
           (long long)n_assign, (long long)MOE_STATIC_MAX_ASSIGN);
  DH_CHECK(experts >= 1 && experts <= MOE_MAX_E, "experts=%d must be in [1, %d]", experts, MOE_MAX_E);
  DH_CHECK(tokens_per_expert && expert_offsets, "null pointer");
  int32_t *hist = nullptr;
  const int rc = moe_static_scratch(&hist);
  if (rc != DH_OK) return rc;
  // Nothing of the table has to start at zero: the histogram kernel writes every (block, expert) entry that the
  // scan and the ranked scatter of this call read, so what an earlier call left behind is never seen.
  return moe_sort_launch(topk_idx, tokens_per_expert, expert_offsets, sorted_idx, dest_row, hist, n_assign, experts,
                         (hipStream_t)stream);
}

static int moe_range_check(int e_lo, int e_hi) { return e_lo >= 0 && e_hi >= e_lo && e_hi <= dh::MOE_MAX_E; }

extern "C" int dh_moe_gather_rows(const void *x, const int32_t *sorted_idx, const float *row_scale, void *permuted,
                                  const int32_t *expert_offsets, int e_lo, int e_hi, int64_t max_rows, int k,
                                  int64_t hidden, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(max_rows >= 0 && hidden >= 0 && k >= 1, "bad shape");
  DH_CHECK(moe_range_check(e_lo, e_hi), "bad expert range [%d, %d)", e_lo, e_hi);
  if (max_rows == 0 || hidden == 0) return DH_OK;
  DH_CHECK(x && sorted_idx && permuted && expert_offsets, "null pointer");
  // rows per workgroup: one (measured, bf16, us for 1 / 2 / 4: 8192 tokens x 4096 11.6 / 11.9 / 12.8; 32768 x 4096
  // 41.2 / 43.4 / 46.9; 8192 x 8192 21.8 / 22.2 / 24.1): more, smaller workgroups get their first loads out sooner
  constexpr int RPB = 1;
  int64_t blocks = cdiv(max_rows, RPB);
  if (blocks > 65536) blocks = 65536;
  DH_DISPATCH_DTYPE(dtype, {
    const int vec_ok = hidden % Vec<T>::N == 0 && aligned16(x) && aligned16(permuted);
    hipLaunchKernelGGL((moe_gather_kernel<T, RPB>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const T *)x, sorted_idx, row_scale, (T *)permuted, expert_offsets, e_lo, e_hi, max_rows, k,
                       hidden, vec_ok);
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

#define DH_SCATTER(KT)                                                                                             \
  hipLaunchKernelGGL((moe_scatter_kernel<T, TPB, KT>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, \
                     (const T *)y, dest_row, gates, (T *)out, expert_offsets, e_lo, e_hi, tokens, k, hidden, vec_ok)

extern "C" int dh_moe_scatter_rows(const void *y, const int32_t *dest_row, const float *gates, void *out,
                                   const int32_t *expert_offsets, int e_lo, int e_hi, int64_t tokens, int k,
                                   int64_t hidden, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(tokens >= 0 && hidden >= 0, "bad shape");
  DH_CHECK(k >= 1 && k <= MOE_MAX_K, "k=%d must be in [1, %d]", k, MOE_MAX_K);
  DH_CHECK(moe_range_check(e_lo, e_hi), "bad expert range [%d, %d)", e_lo, e_hi);
  if (tokens == 0 || hidden == 0) return DH_OK;
  DH_CHECK(dest_row && out && expert_offsets, "null pointer");
  // tokens per workgroup: one (same measurement: 16.1 / 17.2 us at 8192 x 4096, 71.9 / 79.0 at 32768 x 4096)
  constexpr int TPB = 1;
  int64_t blocks = cdiv(tokens, TPB);
  if (blocks > 65536) blocks = 65536;
  DH_DISPATCH_DTYPE(dtype, {
    const int vec_ok = hidden % Vec<T>::N == 0 && aligned16(y) && aligned16(out);
    if (k <= 1) DH_SCATTER(1);
    else if (k <= 2) DH_SCATTER(2);
    else if (k <= 4) DH_SCATTER(4);
    else DH_SCATTER(8);
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_moe_gate_grad(const void *dout, const void *y, const int32_t *dest_row, float *dgates,
                                const int32_t *expert_offsets, int e_lo, int e_hi, int64_t tokens, int k,
                                int64_t hidden, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(tokens >= 0 && hidden >= 0 && k >= 1, "bad shape");
  DH_CHECK(moe_range_check(e_lo, e_hi), "bad expert range [%d, %d)", e_lo, e_hi);
  if (tokens == 0) return DH_OK;
  DH_CHECK(dout && dest_row && dgates && expert_offsets, "null pointer");
  int64_t blocks = tokens * k < 65536 ? tokens * k : 65536;
  DH_DISPATCH_DTYPE(dtype, {
    const int vec_ok = hidden % Vec<T>::N == 0 && aligned16(dout) && aligned16(y);
    hipLaunchKernelGGL((moe_gate_grad_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const T *)dout, (const T *)y, dest_row, dgates, expert_offsets, e_lo, e_hi, tokens, k, hidden,
                       vec_ok);
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

// Head block: vocab-parallel word embedding, vocab-parallel cross entropy, masked mean loss.
//
// All three are HBM-bound.  The reference builds the cross entropy from a dozen full-size torch ops
// (max, subtract, gather, exp, sum, divide, ... in dhellam/operators/loss.py:15-127); here a row of
// logits is read ONCE, held in registers while its maximum, exponential sum and target logit are
// formed, and the softmax (or, in the backward, the gradient) is written from those registers.
// Arithmetic is fp32 whatever the storage type.
#include "common.h"

namespace dh {

namespace {

template <int BT> __device__ __forceinline__ float block_max(float v, float *red) {
  v = wave_max(v);
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int i = 1; i < BT / 64; ++i) t = fmaxf(t, red[i]);
  return t;
}

constexpr float LOG2E = 1.4426950408889634f;

// A row of `cols` elements as seen by one thread of a BT-wide block: up to NV 16-byte vectors kept in
// registers (vector i of the thread is vector i * BT + tid of the row), the rest of the row (long rows,
// the cols % N tail, and rows whose pitch breaks 16-byte alignment) visited from memory each time.
// Column arithmetic is 32-bit and nothing per element depends on the column: with a 64-bit column
// compare per element the backward kernel was bound by the vector ALU, not by memory (2.8 TB/s).
template <typename T, int BT, int NV> struct RowView {
  static constexpr int N = Vec<T>::N;
  const T *row;
  int cols, nvec;           // nvec: whole aligned vectors in the row (0 when the row is not 16-byte aligned)
  Vec<T> held[NV];

  __device__ __forceinline__ void load(const T *r, int c, bool vec_ok) {
    row = r; cols = c; nvec = vec_ok ? c / N : 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = i * BT + (int)threadIdx.x;
      if (v < nvec) held[i] = ldg(row + (int64_t)v * N);
    }
  }
  // f(value) over the part of this thread's share that sits in registers
  template <typename F> __device__ __forceinline__ void for_each_held(F f) const {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = i * BT + (int)threadIdx.x;
      if (v < nvec) {
#pragma unroll
        for (int e = 0; e < N; ++e) f(to_f(held[i].v[e]));
      }
    }
  }
  // ... and over the part that is read from memory on every visit
  template <typename F> __device__ __forceinline__ void for_each_streamed(F f) const {
    constexpr int U = 4;                     // vectors in flight per thread
    int v = NV * BT + (int)threadIdx.x;
    for (; v + (U - 1) * BT < nvec; v += U * BT) {
      Vec<T> x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = ldg(row + (int64_t)(v + u * BT) * N);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int e = 0; e < N; ++e) f(to_f(x[u].v[e]));
    }
    for (; v < nvec; v += BT) {
      const Vec<T> x = ldg(row + (int64_t)v * N);
#pragma unroll
      for (int e = 0; e < N; ++e) f(to_f(x.v[e]));
    }
    for (int c = nvec * N + (int)threadIdx.x; c < cols; c += BT) f(to_f(row[c]));
  }
  template <typename F> __device__ __forceinline__ void for_each(F f) const {
    for_each_held(f);
    for_each_streamed(f);
  }
  // out[c] = g(value) for every column; same traversal, vector stores where the loads were vectors
  // (the caller enables vectors only when `out` is as aligned as the row: a run-time choice between a vector
  // store and element stores of the same values gets merged by the compiler into the element stores)
  template <typename G> __device__ __forceinline__ void map_to(T *out, G g) const {
    auto emit = [&](int v, const Vec<T> &x) {
      Vec<T> o;
#pragma unroll
      for (int e = 0; e < N; ++e) o.v[e] = from_f<T>(g(to_f(x.v[e])));
      stg(out + (int64_t)v * N, o);
    };
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = i * BT + (int)threadIdx.x;
      if (v < nvec) emit(v, held[i]);
    }
    constexpr int U = 4;
    int v = NV * BT + (int)threadIdx.x;
    for (; v + (U - 1) * BT < nvec; v += U * BT) {
      Vec<T> x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = ldg(row + (int64_t)(v + u * BT) * N);
#pragma unroll
      for (int u = 0; u < U; ++u) emit(v + u * BT, x[u]);
    }
    for (; v < nvec; v += BT) emit(v, ldg(row + (int64_t)v * N));
    for (int c = nvec * N + (int)threadIdx.x; c < cols; c += BT) out[c] = from_f<T>(g(to_f(row[c])));
  }
};

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }   // x <= 0 here

}  // namespace

// ---- cross entropy forward --------------------------------------------------------------------------
// One block per row.  Outputs per row: loss, row maximum, sum of exp(x - max), and optionally the target
// logit minus the maximum (0 when the target lies outside [vocab_start, vocab_start + cols)), the mask of
// such targets, the local target index, and the softmax row.  With tensor parallelism the three
// statistics are what a rank contributes to the all-reduces of loss.py:22-24,52-56,61-66.
template <typename T, int BT, int NV>
__global__ void __launch_bounds__(BT) ce_fwd_kernel(const T *__restrict__ logits, const int64_t *__restrict__ target,
                                                    int64_t cols, int64_t ld, int64_t vocab_start, float smoothing,
                                                    float *__restrict__ loss, float *__restrict__ row_max,
                                                    float *__restrict__ sum_exp, float *__restrict__ predicted,
                                                    T *__restrict__ softmax, int64_t ld_sm, uint8_t *__restrict__ tmask,
                                                    int64_t *__restrict__ mtarget, bool vec) {
  __shared__ float red[BT / 64];
  const int64_t r = blockIdx.x;
  RowView<T, BT, NV> rv;
  rv.load(logits + r * ld, (int)cols, vec);
  // The registers are visited twice (maximum, then the exponentials against the block's maximum).  What does not
  // fit in them (rows beyond 16384 logits) is read ONCE, with a running maximum ms and a sum ss of exp(x - ms)
  // that is rescaled whenever ms moves, and joined afterwards: sum += ss * exp(ms - m).
  float m = -INFINITY, sx = 0.f, ms = -INFINITY, ss = 0.f;
  if (smoothing > 0.f) rv.for_each_held([&](float x) { m = fmaxf(m, x); sx += x; });   // sum of x only feeds the smoothing term
  else rv.for_each_held([&](float x) { m = fmaxf(m, x); });
  rv.for_each_streamed([&](float x) {
    // (x - m) first: the difference of two close numbers is exact, the product with log2(e) then errs by
    // one rounding of a small number (x * log2(e) - m * log2(e) would lose |x| * 2^-24 of the exponent).
    const float mn = fmaxf(ms, x);
    if (mn > -INFINITY)                      // (a -inf logit before any finite one contributes nothing)
      ss = ss * exp2_fast((ms - mn) * LOG2E) + exp2_fast((x - mn) * LOG2E);   // ms = -inf at first: 0 * exp2(-inf) = 0
    ms = mn;
    sx += x;
  });
  m = block_max<BT>(fmaxf(m, ms), red);
  float s = ms > -INFINITY ? ss * exp2_fast((ms - m) * LOG2E) : 0.f;
  rv.for_each_held([&](float x) { s += exp2_fast((x - m) * LOG2E); });
  s = block_sum<BT>(s, red);
  if (smoothing > 0.f) sx = block_sum<BT>(sx, red);
  const int64_t t = target[r] - vocab_start;
  const bool outside = t < 0 || t >= cols;
  const int64_t mt = outside ? 0 : t;
  if (threadIdx.x == 0) {
    const float pred = outside ? 0.f : to_f(rv.row[mt]) - m;
    const float ls = logf(s);
    float l = ls - pred;
    // mean of log softmax over the row = mean(x) - max - log(sum)
    if (smoothing > 0.f) l = (1.f - smoothing) * l - smoothing * (sx / (float)cols - m - ls);
    loss[r] = l;
    row_max[r] = m;
    sum_exp[r] = s;
    if (predicted) predicted[r] = pred;
    if (tmask) tmask[r] = outside ? 1 : 0;
    if (mtarget) mtarget[r] = mt;
  }
  if (softmax) {
    const float inv = 1.f / s;
    rv.map_to(softmax + r * ld_sm, [&](float x) { return exp2_fast((x - m) * LOG2E) * inv; });
  }
}

// ---- cross entropy backward -------------------------------------------------------------------------
// grad = (softmax - onehot(target) * (1 - smoothing) * inside - smoothing / cols) * dout[row]
// (loss.py:99-127).  FROM_LOGITS: src holds the logits and the softmax is recomputed from the saved
// row statistics; otherwise src holds the softmax.  grad may alias src (each element is read, then
// written, by the same thread).
template <typename T, int BT, int NV, bool FROM_LOGITS>
__global__ void __launch_bounds__(BT) ce_bwd_kernel(const T *src, int64_t ld_src, const float *__restrict__ row_max,
                                                    const float *__restrict__ sum_exp,
                                                    const int64_t *__restrict__ target, const float *__restrict__ dout,
                                                    int64_t cols, int64_t vocab_start, float smoothing, T *grad,
                                                    int64_t ld_grad, bool vec) {
  const int64_t r = blockIdx.x;
  RowView<T, BT, NV> rv;
  rv.load(src + r * ld_src, (int)cols, vec);
  const int64_t t = target[r] - vocab_start;
  const bool outside = t < 0 || t >= cols;
  const int64_t mt = outside ? 0 : t;
  const float all = smoothing > 0.f ? smoothing / (float)cols : 0.f;
  const float d = dout[r];
  float m = 0.f, inv = 1.f;
  if (FROM_LOGITS) { m = row_max[r]; inv = 1.f / sum_exp[r]; }
  const float k = inv * d, c0 = all * d;
  // Nothing per element depends on the column: the target's element is computed once, by thread 0, from the
  // source value read BEFORE the row is overwritten (grad may be src), and stored after the row.
  float at_target = 0.f;
  if (threadIdx.x == 0 && !outside) {
    const float x = to_f(rv.row[mt]);
    const float p = FROM_LOGITS ? exp2_fast((x - m) * LOG2E) * inv : x;
    at_target = (p - (1.f - smoothing) - all) * d;
  }
  __syncthreads();                           // ... and before any other wavefront's stores can reach that element
  T *out = grad + r * ld_grad;
  if (FROM_LOGITS) rv.map_to(out, [&](float x) { return fmaf(exp2_fast((x - m) * LOG2E), k, -c0); });
  else rv.map_to(out, [&](float x) { return fmaf(x, d, -c0); });
  __syncthreads();                           // the row's stores are complete before the target element is replaced
  if (threadIdx.x == 0 && !outside) out[mt] = from_f<T>(at_target);
}

// ---- word embedding ------------------------------------------------------------------------------------
// out[i] = vocab[ids[i] - vocab_start], zero rows for ids outside this rank's slice (embedding.py:16-39).
template <typename T>
__global__ void __launch_bounds__(256) embedding_fwd_kernel(const T *__restrict__ vocab, const int64_t *__restrict__ ids,
                                                            int64_t hidden, int64_t vocab_rows, int64_t vocab_start,
                                                            T *__restrict__ out) {
  constexpr int N = Vec<T>::N;
  const int64_t i = blockIdx.x;
  const int64_t v = ids[i] - vocab_start;
  const bool inside = v >= 0 && v < vocab_rows;
  const T *src = vocab + (inside ? v : 0) * hidden;
  T *dst = out + i * hidden;
  for (int64_t c = (int64_t)threadIdx.x * N; c < hidden; c += 256 * N) {
    Vec<T> x;
    if (inside) {
      x = ldg(src + c);
    } else {
#pragma unroll
      for (int e = 0; e < N; ++e) x.v[e] = from_f<T>(0.f);
    }
    stg(dst + c, x);
  }
}

// dvocab[v] += sum of dout over the positions whose id is vocab_start + v, in position order: the block of
// the FIRST position holding an id sums all of that id's rows in fp32 and adds the total once, so the result
// does not depend on scheduling and needs no atomics.  Every block scans the id list (n * 8 bytes, from L2):
// quadratic in n, sized for one micro-batch of token ids (4096: 134 MB of L2 reads in all).
// blockIdx.y selects a block of 256 * N * CV columns, held in registers across the scan.
template <typename T, typename TG>
__global__ void __launch_bounds__(256) embedding_bwd_kernel(const T *__restrict__ dout, const int64_t *__restrict__ ids,
                                                            int64_t n, int64_t hidden, int64_t vocab_rows,
                                                            int64_t vocab_start, TG *__restrict__ dvocab) {
  constexpr int N = Vec<T>::N, CV = 4;
  __shared__ int64_t dup[256];
  __shared__ int wcount[4];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int64_t i = blockIdx.x;
  const int64_t id = ids[i];
  const int64_t v = id - vocab_start;
  if (v < 0 || v >= vocab_rows) return;
  int earlier = 0;
  for (int64_t j = tid; j < i; j += 256) earlier |= ids[j] == id;
  if (__syncthreads_or(earlier)) return;     // an earlier position owns this id

  const int64_t c0 = (int64_t)blockIdx.y * (256 * N * CV) + (int64_t)tid * N;
  float acc[CV][N];
#pragma unroll
  for (int q = 0; q < CV; ++q)
#pragma unroll
    for (int e = 0; e < N; ++e) acc[q][e] = 0.f;
  for (int64_t j0 = i; j0 < n; j0 += 256) {
    // ordered compaction of the matching positions of this chunk
    const int64_t j = j0 + tid;
    const bool match = j < n && ids[j] == id;
    const unsigned long long bal = __ballot(match);
    __syncthreads();                         // the previous chunk's dup[] has been consumed
    if (lane == 0) wcount[w] = __popcll(bal);
    __syncthreads();
    int base = 0, total = 0;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      if (x < w) base += wcount[x];
      total += wcount[x];
    }
    if (match) dup[base + __popcll(bal & ((1ull << lane) - 1ull))] = j;
    __syncthreads();
    for (int k = 0; k < total; ++k) {
      const T *row = dout + dup[k] * hidden;
#pragma unroll
      for (int q = 0; q < CV; ++q) {
        const int64_t c = c0 + (int64_t)q * 256 * N;
        if (c < hidden) {
          const Vec<T> x = ldg(row + c);
#pragma unroll
          for (int e = 0; e < N; ++e) acc[q][e] += to_f(x.v[e]);
        }
      }
    }
  }
#pragma unroll
  for (int q = 0; q < CV; ++q) {
    const int64_t c = c0 + (int64_t)q * 256 * N;
    if (c < hidden) {
      TG *g = dvocab + v * hidden + c;
#pragma unroll
      for (int e = 0; e < N; ++e) g[e] = from_f<TG>(to_f(g[e]) + acc[q][e]);
    }
  }
}

// ---- masked mean ---------------------------------------------------------------------------------------
// out[0] = scale * sum(x * mask) / sum(mask), out[1] = sum(mask) (loss.py:131-153 with scale =
// loss_scale / num_microbatch).  One block, fixed summation order.
__global__ void __launch_bounds__(1024) masked_mean_fwd_kernel(const float *__restrict__ x, const float *__restrict__ mask,
                                                               int64_t n, float scale, float *__restrict__ out) {
  __shared__ float red[16];
  float a = 0.f, b = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += 1024) {
    const float mk = mask[i];
    a += x[i] * mk;
    b += mk;
  }
  a = block_sum<1024>(a, red);
  b = block_sum<1024>(b, red);
  if (threadIdx.x == 0) {
    out[0] = a / b * scale;
    out[1] = b;
  }
}

// grad[i] = dout * scale * mask[i] / sum(mask)
__global__ void __launch_bounds__(256) masked_mean_bwd_kernel(const float *__restrict__ mask,
                                                              const float *__restrict__ mask_sum, int64_t n, float scale,
                                                              float *__restrict__ grad) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) grad[i] = mask[i] / mask_sum[0] * scale;
}

}  // namespace dh

using namespace dh;

namespace {
bool row_vec_ok(const void *p, int64_t ld, int dtype) {
  const int64_t n = 16 / (int64_t)dtype_size(dtype);
  return aligned16(p) && ld % n == 0;
}
}  // namespace

extern "C" int dh_cross_entropy_fwd(const void *logits, const int64_t *target, int64_t rows, int64_t cols, int64_t ld,
                                    int64_t vocab_start, float label_smoothing, int dtype, float *loss, float *row_max,
                                    float *sum_exp, float *predicted, void *softmax, int64_t ld_softmax,
                                    uint8_t *target_mask, int64_t *masked_target, void *stream) {
  DH_CHECK(rows >= 0 && cols > 0 && ld >= cols, "rows=%lld cols=%lld ld=%lld", (long long)rows, (long long)cols,
           (long long)ld);
  DH_CHECK(label_smoothing >= 0.f && label_smoothing < 1.f, "label_smoothing %g outside [0, 1)", label_smoothing);
  DH_CHECK(label_smoothing == 0.f || cols > 1, "label smoothing needs more than one class");
  if (rows == 0) return DH_OK;
  DH_CHECK(logits && target && loss && row_max && sum_exp, "null pointer");
  DH_CHECK(!softmax || ld_softmax >= cols, "ld_softmax=%lld < cols", (long long)ld_softmax);
  {
    const char *a = (const char *)logits, *b = (const char *)softmax;
    const int64_t e = (int64_t)dtype_size(dtype);
    DH_CHECK(!softmax || a + ((rows - 1) * ld + cols) * e <= b || b + ((rows - 1) * ld_softmax + cols) * e <= a,
             "softmax must not overlap the logits");
  }
  DH_CHECK(rows < (1ll << 31) && cols < (1ll << 31), "too many rows or columns");
  const float smoothing = label_smoothing > 0.f ? label_smoothing * (float)cols / (float)(cols - 1) : 0.f;
  // vector accesses only when the logits and (if asked for) the softmax rows are all 16-byte aligned
  const bool vec = row_vec_ok(logits, ld, dtype) && (!softmax || row_vec_ok(softmax, ld_softmax, dtype));
  DH_DISPATCH_DTYPE(dtype, {
    // 256 threads per row holding 16384 logits in registers (128 bytes per thread for 16-bit types, 256 for fp32;
    // an fp32 row half held and half re-read ran at 4.5 instead of 6.4 TB/s).  With 1024 threads and 2 rows per
    // CU the kernel ran at half the rate; 128 threads per 16-bit row were slower as well (4.0 against 4.8 TB/s).
    constexpr int BT = 256, NV = sizeof(T) == 4 ? 16 : 8;
    hipLaunchKernelGGL((ce_fwd_kernel<T, BT, NV>), dim3((unsigned)rows), dim3(BT), 0, (hipStream_t)stream,
                       (const T *)logits, target, cols, ld, vocab_start, smoothing, loss, row_max, sum_exp, predicted,
                       (T *)softmax, ld_softmax, target_mask, masked_target, vec);
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_cross_entropy_bwd(const void *src, int64_t ld_src, int from_logits, const float *row_max,
                                    const float *sum_exp, const int64_t *target, const float *dout, int64_t rows,
                                    int64_t cols, int64_t vocab_start, float label_smoothing, int dtype, void *grad,
                                    int64_t ld_grad, void *stream) {
  DH_CHECK(rows >= 0 && cols > 0 && ld_src >= cols && ld_grad >= cols, "rows=%lld cols=%lld ld_src=%lld ld_grad=%lld",
           (long long)rows, (long long)cols, (long long)ld_src, (long long)ld_grad);
  DH_CHECK(label_smoothing >= 0.f && label_smoothing < 1.f, "label_smoothing %g outside [0, 1)", label_smoothing);
  DH_CHECK(label_smoothing == 0.f || cols > 1, "label smoothing needs more than one class");
  if (rows == 0) return DH_OK;
  DH_CHECK(src && target && dout && grad, "null pointer");
  DH_CHECK(!from_logits || (row_max && sum_exp), "recomputing the softmax needs row_max and sum_exp");
  {
    const char *a = (const char *)src, *b = (const char *)grad;
    const int64_t e = (int64_t)dtype_size(dtype);
    DH_CHECK((a == b && ld_grad == ld_src) || a + ((rows - 1) * ld_src + cols) * e <= b ||
                 b + ((rows - 1) * ld_grad + cols) * e <= a,
             "grad is either src itself (same pitch) or does not overlap it");
  }
  DH_CHECK(rows < (1ll << 31) && cols < (1ll << 31), "too many rows or columns");
  const float smoothing = label_smoothing > 0.f ? label_smoothing * (float)cols / (float)(cols - 1) : 0.f;
  const bool vec = row_vec_ok(src, ld_src, dtype) && row_vec_ok(grad, ld_grad, dtype);
  DH_DISPATCH_DTYPE(dtype, {
    // 256 threads per row holding 16384 logits in registers (128 bytes per thread for 16-bit types, 256 for fp32;
    // an fp32 row half held and half re-read ran at 4.5 instead of 6.4 TB/s).  With 1024 threads and 2 rows per
    // CU the kernel ran at half the rate; 128 threads per 16-bit row were slower as well (4.0 against 4.8 TB/s).
    constexpr int BT = 256, NV = sizeof(T) == 4 ? 16 : 8;
    if (from_logits)
      hipLaunchKernelGGL((ce_bwd_kernel<T, BT, NV, true>), dim3((unsigned)rows), dim3(BT), 0, (hipStream_t)stream,
                         (const T *)src, ld_src, row_max, sum_exp, target, dout, cols, vocab_start, smoothing, (T *)grad,
                         ld_grad, vec);
    else
      hipLaunchKernelGGL((ce_bwd_kernel<T, BT, NV, false>), dim3((unsigned)rows), dim3(BT), 0, (hipStream_t)stream,
                         (const T *)src, ld_src, row_max, sum_exp, target, dout, cols, vocab_start, smoothing, (T *)grad,
                         ld_grad, vec);
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_embedding_fwd(const void *vocab, const int64_t *ids, int64_t n, int64_t hidden, int64_t vocab_rows,
                                int64_t vocab_start, int dtype, void *out, void *stream) {
  DH_CHECK(n >= 0 && hidden > 0 && vocab_rows > 0, "n=%lld hidden=%lld vocab_rows=%lld", (long long)n, (long long)hidden,
           (long long)vocab_rows);
  if (n == 0) return DH_OK;
  DH_CHECK(vocab && ids && out, "null pointer");
  DH_CHECK(hidden % (16 / (int64_t)dtype_size(dtype)) == 0 && aligned16(vocab) && aligned16(out),
           "hidden=%lld must fill whole 16-byte vectors and the tensors must be 16-byte aligned", (long long)hidden);
  DH_CHECK(n < (1ll << 31), "too many ids");
  DH_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((embedding_fwd_kernel<T>), dim3((unsigned)n), dim3(256), 0,
                                              (hipStream_t)stream, (const T *)vocab, ids, hidden, vocab_rows,
                                              vocab_start, (T *)out));
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_embedding_bwd(const void *dout, const int64_t *ids, int64_t n, int64_t hidden, int64_t vocab_rows,
                                int64_t vocab_start, int dtype, void *dvocab, int dvocab_dtype, void *stream) {
  DH_CHECK(n >= 0 && hidden > 0 && vocab_rows > 0, "n=%lld hidden=%lld vocab_rows=%lld", (long long)n, (long long)hidden,
           (long long)vocab_rows);
  if (n == 0) return DH_OK;
  DH_CHECK(dout && ids && dvocab, "null pointer");
  DH_CHECK(hidden % (16 / (int64_t)dtype_size(dtype)) == 0 && aligned16(dout),
           "hidden=%lld must fill whole 16-byte vectors and dout must be 16-byte aligned", (long long)hidden);
  DH_CHECK(dvocab_dtype == dtype || dvocab_dtype == DH_F32, "dvocab is fp32 or of dout's type");
  DH_CHECK(n < (1ll << 31), "too many ids");
  DH_DISPATCH_DTYPE(dtype, {
    const dim3 grid((unsigned)n, (unsigned)cdiv(hidden, 256 * (16 / (int64_t)sizeof(T)) * 4));
    if (dvocab_dtype == DH_F32)
      hipLaunchKernelGGL((embedding_bwd_kernel<T, float>), grid, dim3(256), 0, (hipStream_t)stream,
                         (const T *)dout, ids, n, hidden, vocab_rows, vocab_start, (float *)dvocab);
    else
      hipLaunchKernelGGL((embedding_bwd_kernel<T, T>), grid, dim3(256), 0, (hipStream_t)stream,
                         (const T *)dout, ids, n, hidden, vocab_rows, vocab_start, (T *)dvocab);
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_masked_mean_fwd(const float *x, const float *mask, int64_t n, float scale, float *out, void *stream) {
  DH_CHECK(n > 0, "n=%lld", (long long)n);
  DH_CHECK(x && mask && out, "null pointer");
  hipLaunchKernelGGL(masked_mean_fwd_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, x, mask, n, scale, out);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_masked_mean_bwd(const float *mask, const float *mask_sum, int64_t n, float scale, float *grad,
                                  void *stream) {
  DH_CHECK(n > 0, "n=%lld", (long long)n);
  DH_CHECK(mask && mask_sum && grad, "null pointer");
  hipLaunchKernelGGL(masked_mean_bwd_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream, mask,
                     mask_sum, n, scale, grad);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

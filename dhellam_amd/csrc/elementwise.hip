// Streaming elementwise kernels: SwiGLU forward/backward, residual add, and the
// two legacy kernels of the binding surface (tanh-GELU, bias-mask-add).
// All are HBM-bound: 16-byte accesses, several independent loads in flight per
// lane, fp32 math, one rounding on store.
#include "common.h"

namespace dh {

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + __expf(-x)); }
// out = silu(gate) * up for one element, every operation rounded by itself and the last product kept apart from
// the caller's conversion (the kernels that use it must give the same bits).
__device__ __forceinline__ float swiglu_value(float g, float u) {
#pragma clang fp contract(off)
  float o = g * sigmoidf_(g) * u;
  asm("" : "+v"(o));
  return o;
}
// d(gate) and d(up) of out = silu(gate) * up for one element, every operation rounded by itself (no fused multiply-add: the
// kernels that use it must give the same bits, whatever the compiler would fuse around each call).
__device__ __forceinline__ void swiglu_grad(float y1, float y2, float gg, float &d1, float &d2) {
#pragma clang fp contract(off)
  const float s = sigmoidf_(y1);
  const float u = 1.0f + y1 * (1.0f - s);
  d1 = gg * s * u * y2;
  d2 = gg * (y1 * s);
  // keeps the last product apart from the caller's conversion to 16 bits (one instruction can do both, rounding
  // once instead of twice, and whether the compiler picks it depends on the code around the call)
  asm("" : "+v"(d1), "+v"(d2));
}

// One "item" = one 16-byte vector of the output row; rows x fv items in total.
// Item mapping of the streaming kernels: blocked = a workgroup's UNROLL vectors per lane are 256
// apart (one contiguous 4 KB * UNROLL run per workgroup per trip); otherwise a grid stride apart.
#ifndef DH_EW_BLOCKED
#define DH_EW_BLOCKED 1
#endif
#ifndef DH_EW_MAXGRID
#define DH_EW_MAXGRID 65536
#endif

// IDX: the type the item index is computed in.  Splitting an item index into (row, column) is a division by the
// run-time row length, and it stands in front of a workgroup's first load: in 64 bits it is some forty
// instructions per vector, in 32 bits (whenever the item count allows) a handful.
template <typename T, int UNROLL, bool NT, typename IDX>
__global__ void __launch_bounds__(256)
swiglu_fwd_kernel(const T *__restrict__ y, T *__restrict__ out, int64_t nitems_, int fv_) {
  constexpr int N = Vec<T>::N;
  const IDX nitems = (IDX)nitems_, fv = (IDX)fv_;
  const IDX stride = (IDX)gridDim.x * 256;
  const IDX ustride = DH_EW_BLOCKED ? 256 : stride;
  IDX it = (IDX)blockIdx.x * (DH_EW_BLOCKED ? 256 * UNROLL : 256) + threadIdx.x;
  for (; it < nitems; it += stride * UNROLL) {
    Vec<T> a[UNROLL], b[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const IDX id = it + u * ustride;
      if (id < nitems) {
        const IDX r = id / fv;
        const int c = (int)(id - r * fv);
        const T *row = y + (int64_t)r * (2 * (int64_t)fv * N);
        a[u] = ldg_s<NT>(row + (int64_t)c * N);
        b[u] = ldg_s<NT>(row + ((int64_t)fv + c) * N);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const IDX id = it + u * ustride;
      if (id < nitems) {
        Vec<T> o;
#pragma unroll
        for (int j = 0; j < N; ++j) {
          o.v[j] = from_f<T>(swiglu_value(to_f(a[u].v[j]), to_f(b[u].v[j])));
        }
        stg_s<NT>(out + (int64_t)id * N, o);
      }
    }
  }
}

template <typename T, int UNROLL, bool NT, typename IDX>
__global__ void __launch_bounds__(256)
swiglu_bwd_kernel(const T *__restrict__ g, const T *__restrict__ y, T *__restrict__ dy, int64_t nitems_, int fv_) {
  constexpr int N = Vec<T>::N;
  const IDX nitems = (IDX)nitems_, fv = (IDX)fv_;
  const IDX stride = (IDX)gridDim.x * 256;
  const IDX ustride = DH_EW_BLOCKED ? 256 : stride;
  IDX it = (IDX)blockIdx.x * (DH_EW_BLOCKED ? 256 * UNROLL : 256) + threadIdx.x;
  for (; it < nitems; it += stride * UNROLL) {
    Vec<T> a[UNROLL], b[UNROLL], gv[UNROLL];
    IDX rr[UNROLL];
    int cc[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const IDX id = it + u * ustride;
      if (id < nitems) {
        const IDX r = id / fv;
        const int c = (int)(id - r * fv);
        rr[u] = r;
        cc[u] = c;
        const T *row = y + (int64_t)r * (2 * (int64_t)fv * N);
        a[u] = ldg_s<NT>(row + (int64_t)c * N);
        b[u] = ldg_s<NT>(row + ((int64_t)fv + c) * N);
        gv[u] = ldg_s<NT>(g + (int64_t)id * N);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const IDX id = it + u * ustride;
      if (id < nitems) {
        const IDX r = rr[u];
        const int c = cc[u];
        Vec<T> d1, d2;
#pragma unroll
        for (int j = 0; j < N; ++j) {
          float v1, v2;
          swiglu_grad(to_f(a[u].v[j]), to_f(b[u].v[j]), to_f(gv[u].v[j]), v1, v2);
          d1.v[j] = from_f<T>(v1);
          d2.v[j] = from_f<T>(v2);
        }
        T *row = dy + (int64_t)r * (2 * (int64_t)fv * N);
        stg_s<NT>(row + (int64_t)c * N, d1);
        stg_s<NT>(row + ((int64_t)fv + c) * N, d2);
      }
    }
  }
}

// SwiGLU forward that also writes its result transposed: out [rows, f] and outT [f, rows] from one read of y.  The
// transpose feeds the weight-gradient GEMM of the projection BEHIND the activation (dW = dY^T out runs fastest with
// one operand transposed, and out is the smaller one there); produced here it costs one more write instead of a
// read and a write of its own.  Same tiling as the backward below: a workgroup takes 64 rows x 128 columns,
// stores them as rows, and passes them through LDS to store them as columns, 8 rows per lane.
template <typename T>
__global__ void __launch_bounds__(256)
swiglu_fwd_t_kernel(const T *__restrict__ y, T *__restrict__ out, T *__restrict__ outt, int64_t rows, int64_t f,
                    int64_t ld_t) {
  constexpr int N = Vec<T>::N;                      // 8
  constexpr int TR = 64, TC = 128, PITCH = TC * 2 + 4;
  __shared__ __attribute__((aligned(16))) unsigned char tile[TR * PITCH];
  const int64_t r0 = (int64_t)blockIdx.y * TR, c0 = (int64_t)blockIdx.x * TC;
  const int tid = threadIdx.x;
  {
    const int lr = tid >> 4, ch = tid & 15;
    Vec<T> a[4], b[4];
    bool ok[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t r = r0 + lr + 16 * i, c = c0 + ch * N;
      ok[i] = r < rows && c < f;
      if (ok[i]) {
        const T *row = y + r * (2 * f);
        a[i] = ldg(row + c);
        b[i] = ldg(row + f + c);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int rl = lr + 16 * i;
      Vec<T> o;
#pragma unroll
      for (int j = 0; j < N; ++j) o.v[j] = from_f<T>(ok[i] ? swiglu_value(to_f(a[i].v[j]), to_f(b[i].v[j])) : 0.f);
      if (ok[i]) stg(out + (r0 + rl) * f + c0 + ch * N, o);
      const uint32_t *s1 = reinterpret_cast<const uint32_t *>(&o);      // rows are 4-byte aligned only: dword stores
      uint32_t *t1 = reinterpret_cast<uint32_t *>(tile + rl * PITCH + ch * 16);
#pragma unroll
      for (int q = 0; q < 4; ++q) t1[q] = s1[q];
    }
  }
  __syncthreads();
  const int lane = tid & 63, w = tid >> 6;
  const int rb = lane & 7, cl = lane >> 3;            // 8-row block, column within the step
#pragma unroll
  for (int s2 = 0; s2 < 4; ++s2) {
    const int col = 32 * w + 8 * s2 + cl;
    const unsigned char *src = tile + (8 * rb) * PITCH + col * 2;
    Vec<T> o;
#pragma unroll
    for (int j = 0; j < N; ++j) o.v[j] = *reinterpret_cast<const T *>(src + j * PITCH);
    if (c0 + col < f && r0 + 8 * rb < rows) stg(outt + (c0 + col) * ld_t + r0 + 8 * rb, o);
  }
}

// SwiGLU backward that also writes the gradient transposed: dy [rows, 2f] and dyT [2f, rows] from one read of g and
// y.  The transpose feeds the weight-gradient GEMM of the projection in front of the activation (dW = dy^T x runs
// fastest with dy^T row-major); produced here it costs one more write instead of a read and a write of its own.
// A workgroup takes 64 rows x 128 columns of g: it computes the 64 x 128 tiles of d(gate) and d(up), stores them
// as rows, and passes them through LDS (rows of 65 dwords, so 8-row steps land 8 banks apart) to store them as
// columns: every lane gathers 8 consecutive rows of one column and writes them as 16 contiguous bytes, the 8
// lanes of a column adjacent, i.e. whole 128-byte lines of dyT per store instruction.
template <typename T>
__global__ void __launch_bounds__(256)
swiglu_bwd_t_kernel(const T *__restrict__ g, const T *__restrict__ y, T *__restrict__ dy, T *__restrict__ dyt,
                    int64_t rows, int64_t f, int64_t ld_t) {
  constexpr int N = Vec<T>::N;                      // 8
  constexpr int TR = 64, TC = 128, PITCH = TC * 2 + 4;
  __shared__ __attribute__((aligned(16))) unsigned char tile[2][TR * PITCH];
  const int64_t r0 = (int64_t)blockIdx.y * TR, c0 = (int64_t)blockIdx.x * TC;
  const int tid = threadIdx.x;
  {
    const int lr = tid >> 4, ch = tid & 15;
    Vec<T> a[4], b[4], gv[4];
    bool ok[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t r = r0 + lr + 16 * i, c = c0 + ch * N;
      ok[i] = r < rows && c < f;
      if (ok[i]) {
        const T *row = y + r * (2 * f);
        a[i] = ldg(row + c);
        b[i] = ldg(row + f + c);
        gv[i] = ldg(g + r * f + c);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int rl = lr + 16 * i;
      Vec<T> d1, d2;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        float v1 = 0.f, v2 = 0.f;
        if (ok[i]) swiglu_grad(to_f(a[i].v[j]), to_f(b[i].v[j]), to_f(gv[i].v[j]), v1, v2);
        d1.v[j] = from_f<T>(v1);
        d2.v[j] = from_f<T>(v2);
      }
      if (ok[i]) {
        T *row = dy + (r0 + rl) * (2 * f);
        stg(row + c0 + ch * N, d1);
        stg(row + f + c0 + ch * N, d2);
      }
      // rows are 4-byte aligned only: dword stores
      const uint32_t *s1 = reinterpret_cast<const uint32_t *>(&d1), *s2 = reinterpret_cast<const uint32_t *>(&d2);
      uint32_t *t1 = reinterpret_cast<uint32_t *>(tile[0] + rl * PITCH + ch * 16);
      uint32_t *t2 = reinterpret_cast<uint32_t *>(tile[1] + rl * PITCH + ch * 16);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        t1[q] = s1[q];
        t2[q] = s2[q];
      }
    }
  }
  __syncthreads();
  const int lane = tid & 63, w = tid >> 6;
  const int rb = lane & 7, cl = lane >> 3;            // 8-row block, column within the step
#pragma unroll
  for (int part = 0; part < 2; ++part)
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
      const int col = 32 * w + 8 * s2 + cl;
      const unsigned char *src = tile[part] + (8 * rb) * PITCH + col * 2;
      Vec<T> o;
#pragma unroll
      for (int j = 0; j < N; ++j) o.v[j] = *reinterpret_cast<const T *>(src + j * PITCH);
      if (c0 + col < f && r0 + 8 * rb < rows) stg(dyt + ((int64_t)part * f + c0 + col) * ld_t + r0 + 8 * rb, o);
    }
}

// Scalar fallbacks (f not a multiple of the vector width, or unaligned pointers).
template <typename T>
__global__ void __launch_bounds__(256)
swiglu_fwd_scalar_kernel(const T *__restrict__ y, T *__restrict__ out, int64_t n, int64_t f) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / f, c = i - r * f;
    const float g = to_f(y[r * 2 * f + c]);
    out[i] = from_f<T>(swiglu_value(g, to_f(y[r * 2 * f + f + c])));
  }
}
template <typename T>
__global__ void __launch_bounds__(256)
swiglu_bwd_scalar_kernel(const T *__restrict__ g, const T *__restrict__ y, T *__restrict__ dy, int64_t n,
                         int64_t f) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / f, c = i - r * f;
    const float y1 = to_f(y[r * 2 * f + c]), y2 = to_f(y[r * 2 * f + f + c]), gg = to_f(g[i]);
    float v1, v2;
    swiglu_grad(y1, y2, gg, v1, v2);
    dy[r * 2 * f + c] = from_f<T>(v1);
    dy[r * 2 * f + f + c] = from_f<T>(v2);
  }
}

enum { EW_ADD = 0, EW_GELU = 1, EW_BMA = 2 };

template <typename T, int OP>
__device__ __forceinline__ float ew_apply(float x, float b, float r, float m) {
  if (OP == EW_ADD) return x + r;
  if (OP == EW_GELU) return x * (0.5f + 0.5f * tanhf(x * (0.79788456f + 0.03567741f * x * x)));
  return m * (x + b) + r;
}

template <typename T, int OP, int UNROLL, bool NT>
__global__ void __launch_bounds__(256)
ew_kernel(const T *__restrict__ x, const T *__restrict__ bias, const T *__restrict__ res, const T *__restrict__ mask,
          T *__restrict__ out, int64_t nvec, int64_t n) {
  constexpr int N = Vec<T>::N;
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t ustride = DH_EW_BLOCKED ? 256 : stride;
  int64_t it = (int64_t)blockIdx.x * (DH_EW_BLOCKED ? 256 * UNROLL : 256) + threadIdx.x;
  for (; it < nvec; it += stride * UNROLL) {
    Vec<T> xv[UNROLL], bv[UNROLL], rv[UNROLL], mv[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t id = it + u * ustride;
      if (id < nvec) {
        xv[u] = ldg_s<NT>(x + id * N);
        if (OP != EW_GELU) rv[u] = ldg_s<NT>(res + id * N);
        if (OP == EW_BMA) {
          bv[u] = ldg_s<NT>(bias + id * N);
          if (mask) mv[u] = ldg_s<NT>(mask + id * N);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t id = it + u * ustride;
      if (id < nvec) {
        Vec<T> o;
#pragma unroll
        for (int j = 0; j < N; ++j) {
          const float m = (OP == EW_BMA && mask) ? to_f(mv[u].v[j]) : 1.0f;
          o.v[j] = from_f<T>(ew_apply<T, OP>(to_f(xv[u].v[j]), OP == EW_BMA ? to_f(bv[u].v[j]) : 0.f,
                                             OP != EW_GELU ? to_f(rv[u].v[j]) : 0.f, m));
        }
        stg_s<NT>(out + id * N, o);
      }
    }
  }
  // tail elements (n % N) and everything when nvec == 0
  const int64_t t0 = nvec * N;
  if (blockIdx.x == 0) {
    for (int64_t i = t0 + threadIdx.x; i < n; i += 256) {
      const float m = (OP == EW_BMA && mask) ? to_f(mask[i]) : 1.0f;
      out[i] = from_f<T>(ew_apply<T, OP>(to_f(x[i]), OP == EW_BMA ? to_f(bias[i]) : 0.f,
                                         OP != EW_GELU ? to_f(res[i]) : 0.f, m));
    }
  }
}

static inline unsigned stream_grid(int64_t items, int per_thread) {
  int64_t b = cdiv(items, 256ll * per_thread);
  if (b < 1) b = 1;
  if (b > DH_EW_MAXGRID) b = DH_EW_MAXGRID;
  return (unsigned)b;
}

template <typename T, int OP>
static int launch_ew(const void *x, const void *bias, const void *res, const void *mask, void *out, int64_t n,
                     hipStream_t st) {
  constexpr int N = Vec<T>::N;
  bool al = aligned16(x) && aligned16(out) && (!bias || aligned16(bias)) && (!res || aligned16(res)) &&
            (!mask || aligned16(mask));
  const int64_t nvec = al ? n / N : 0;
  const int streams = 2 + (bias ? 1 : 0) + (res ? 1 : 0) + (mask ? 1 : 0);
#define L(NT)                                                                                                 \
  hipLaunchKernelGGL((ew_kernel<T, OP, 4, NT>), dim3(stream_grid(nvec, 4)), dim3(256), 0, st, (const T *)x,     \
                     (const T *)bias, (const T *)res, (const T *)mask, (T *)out, nvec, n)
  if (stream_hint(n * (int64_t)sizeof(T) * streams)) L(true); else L(false);
#undef L
  return 0;
}

// nitems 16-byte output vectors; the forward touches 3 of them per item, the backward 5.
// Vectors in flight per lane: measured on [rows, 2 x 3584] bf16 (forward, us at 512 / 4096 / 16384 / 65536 rows):
// one 3.6 / 15.5 / 54.8 / 231, two 3.7 / 16.4 / 56.3 / 222, four 4.2 / 18.5 / 61.4 / 234.  Below a few hundred MB
// more, smaller workgroups win (the whole tensor is in flight at once and what counts is how soon the first loads
// go out); beyond that two vectors per lane do.
template <typename T, int U>
static void launch_swiglu_fwd_u(const T *y, T *out, int64_t nitems, int fv, hipStream_t st) {
  const dim3 grid(stream_grid(nitems, U));
  // 32-bit item arithmetic while an index one trip past the end still fits
  const bool small = nitems + (int64_t)grid.x * 256 * U < (1ll << 32);
#define L(NT, IDX) hipLaunchKernelGGL((swiglu_fwd_kernel<T, U, NT, IDX>), grid, dim3(256), 0, st, y, out, nitems, fv)
  if (stream_hint(3 * 16 * nitems)) { if (small) L(true, uint32_t); else L(true, int64_t); }
  else { if (small) L(false, uint32_t); else L(false, int64_t); }
#undef L
}
template <typename T>
static void launch_swiglu_fwd(const T *y, T *out, int64_t nitems, int fv, hipStream_t st) {
  if (3 * 16 * nitems <= (512ll << 20)) launch_swiglu_fwd_u<T, 1>(y, out, nitems, fv, st);
  else launch_swiglu_fwd_u<T, 2>(y, out, nitems, fv, st);
}
template <typename T, int U>
static void launch_swiglu_bwd_u(const T *g, const T *y, T *dy, int64_t nitems, int fv, hipStream_t st) {
  const dim3 grid(stream_grid(nitems, U));
  const bool small = nitems + (int64_t)grid.x * 256 * U < (1ll << 32);
#define L(NT, IDX) hipLaunchKernelGGL((swiglu_bwd_kernel<T, U, NT, IDX>), grid, dim3(256), 0, st, g, y, dy, nitems, fv)
  if (stream_hint(5 * 16 * nitems)) { if (small) L(true, uint32_t); else L(true, int64_t); }
  else { if (small) L(false, uint32_t); else L(false, int64_t); }
#undef L
}
// (backward, same shapes: one vector per lane 4.4 / 22.8 / 91.3 / 390 us, two 4.9 / 23.5 / 92.8 / 381)
template <typename T>
static void launch_swiglu_bwd(const T *g, const T *y, T *dy, int64_t nitems, int fv, hipStream_t st) {
  if (5 * 16 * nitems <= (768ll << 20)) launch_swiglu_bwd_u<T, 1>(g, y, dy, nitems, fv, st);
  else launch_swiglu_bwd_u<T, 2>(g, y, dy, nitems, fv, st);
}

}  // namespace dh

extern "C" int dh_swiglu_fwd(const void *y, void *out, int64_t rows, int64_t f, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(rows >= 0 && f >= 0, "bad shape rows=%lld f=%lld", (long long)rows, (long long)f);
  if (rows == 0 || f == 0) return DH_OK;
  DH_CHECK(y && out, "null pointer");
  hipStream_t st = (hipStream_t)stream;
  DH_DISPATCH_DTYPE(dtype, {
    constexpr int N = Vec<T>::N;
    if (f % N == 0 && aligned16(y) && aligned16(out) && f / N < (1ll << 31)) {
      const int64_t nitems = rows * (f / N);
      launch_swiglu_fwd<T>((const T *)y, (T *)out, nitems, (int)(f / N), st);
    } else {
      hipLaunchKernelGGL((swiglu_fwd_scalar_kernel<T>), dim3(stream_grid(rows * f, 4)), dim3(256), 0, st,
                         (const T *)y, (T *)out, rows * f, f);
    }
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_swiglu_bwd(const void *g, const void *y, void *dy, int64_t rows, int64_t f, int dtype,
                             void *stream) {
  using namespace dh;
  DH_CHECK(rows >= 0 && f >= 0, "bad shape rows=%lld f=%lld", (long long)rows, (long long)f);
  if (rows == 0 || f == 0) return DH_OK;
  DH_CHECK(g && y && dy, "null pointer");
  hipStream_t st = (hipStream_t)stream;
  DH_DISPATCH_DTYPE(dtype, {
    constexpr int N = Vec<T>::N;
    if (f % N == 0 && aligned16(y) && aligned16(g) && aligned16(dy) && f / N < (1ll << 31)) {
      const int64_t nitems = rows * (f / N);
      launch_swiglu_bwd<T>((const T *)g, (const T *)y, (T *)dy, nitems, (int)(f / N), st);
    } else {
      hipLaunchKernelGGL((swiglu_bwd_scalar_kernel<T>), dim3(stream_grid(rows * f, 4)), dim3(256), 0, st,
                         (const T *)g, (const T *)y, (T *)dy, rows * f, f);
    }
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_swiglu_fwd_t(const void *y, void *out, void *out_t, int64_t rows, int64_t f, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(rows >= 0 && f >= 0, "bad shape rows=%lld f=%lld", (long long)rows, (long long)f);
  if (rows == 0 || f == 0) return DH_OK;
  DH_CHECK(y && out && out_t, "null pointer");
  DH_CHECK(dtype == DH_BF16 || dtype == DH_F16, "16-bit element types only (dtype %d)", dtype);
  DH_CHECK(rows % 8 == 0 && f % 8 == 0, "rows=%lld and f=%lld must be multiples of 8", (long long)rows, (long long)f);
  DH_CHECK(aligned16(y) && aligned16(out) && aligned16(out_t), "pointers must be 16-byte aligned");
  const dim3 grid((unsigned)cdiv(f, 128), (unsigned)cdiv(rows, 64));
  DH_CHECK(grid.y < 65536, "too many rows for one launch");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == DH_BF16)
    hipLaunchKernelGGL((swiglu_fwd_t_kernel<bf16_t>), grid, dim3(256), 0, st, (const bf16_t *)y, (bf16_t *)out,
                       (bf16_t *)out_t, rows, f, rows);
  else
    hipLaunchKernelGGL((swiglu_fwd_t_kernel<f16_t>), grid, dim3(256), 0, st, (const f16_t *)y, (f16_t *)out,
                       (f16_t *)out_t, rows, f, rows);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_swiglu_bwd_t(const void *g, const void *y, void *dy, void *dy_t, int64_t rows, int64_t f, int dtype,
                               void *stream) {
  using namespace dh;
  DH_CHECK(rows >= 0 && f >= 0, "bad shape rows=%lld f=%lld", (long long)rows, (long long)f);
  if (rows == 0 || f == 0) return DH_OK;
  DH_CHECK(g && y && dy && dy_t, "null pointer");
  DH_CHECK(dtype == DH_BF16 || dtype == DH_F16, "16-bit element types only (dtype %d)", dtype);
  DH_CHECK(rows % 8 == 0 && f % 8 == 0, "rows=%lld and f=%lld must be multiples of 8", (long long)rows, (long long)f);
  DH_CHECK(aligned16(y) && aligned16(g) && aligned16(dy) && aligned16(dy_t), "pointers must be 16-byte aligned");
  const dim3 grid((unsigned)cdiv(f, 128), (unsigned)cdiv(rows, 64));
  DH_CHECK(grid.y < 65536, "too many rows for one launch");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == DH_BF16)
    hipLaunchKernelGGL((swiglu_bwd_t_kernel<bf16_t>), grid, dim3(256), 0, st, (const bf16_t *)g, (const bf16_t *)y,
                       (bf16_t *)dy, (bf16_t *)dy_t, rows, f, rows);
  else
    hipLaunchKernelGGL((swiglu_bwd_t_kernel<f16_t>), grid, dim3(256), 0, st, (const f16_t *)g, (const f16_t *)y,
                       (f16_t *)dy, (f16_t *)dy_t, rows, f, rows);
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_residual_add(const void *x, const void *residual, void *out, int64_t n, int dtype,
                               void *stream) {
  using namespace dh;
  DH_CHECK(n >= 0, "n must be >= 0");
  if (n == 0) return DH_OK;
  DH_CHECK(x && residual && out, "null pointer");
  DH_DISPATCH_DTYPE(dtype, { launch_ew<T, EW_ADD>(x, nullptr, residual, nullptr, out, n, (hipStream_t)stream); });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_gelu(const void *x, void *out, int64_t n, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(n >= 0, "n must be >= 0");
  if (n == 0) return DH_OK;
  DH_CHECK(x && out, "null pointer");
  DH_DISPATCH_DTYPE(dtype, { launch_ew<T, EW_GELU>(x, nullptr, nullptr, nullptr, out, n, (hipStream_t)stream); });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_bias_mask_add(const void *x, const void *bias, const void *residual, const void *mask, void *out,
                                int64_t n, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(n >= 0, "n must be >= 0");
  if (n == 0) return DH_OK;
  DH_CHECK(x && bias && residual && out, "null pointer");
  DH_DISPATCH_DTYPE(dtype, { launch_ew<T, EW_BMA>(x, bias, residual, mask, out, n, (hipStream_t)stream); });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

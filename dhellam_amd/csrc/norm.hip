// RMSNorm / LayerNorm forward and backward for gfx950.
//
// Bandwidth-bound: every row is read once with 16-byte loads, kept in
// registers between the statistics pass and the normalise pass, and written
// once.  A row is owned by one wavefront (narrow rows) or by the whole
// 256-thread block (wide rows); reductions are wave64 shuffles plus four LDS
// words.  Backward accumulates dgamma/dbeta per thread-owned column over the
// rows a block walks, stages the per-wave partials through LDS, writes one
// fp32 partial row per block, and a second small kernel reduces the partial
// rows in a fixed order (deterministic, no atomics).
#include "common.h"

namespace dh {

template <typename T, int BT, int TPR, int VPT, bool LN, bool NT, bool RES>
__global__ void __launch_bounds__(BT)
norm_fwd_kernel(const T *__restrict__ x, const T *__restrict__ residual, T *__restrict__ sum_out,
                const T *__restrict__ gamma, const T *__restrict__ beta,
                T *__restrict__ y, float *__restrict__ mu_out, float *__restrict__ rs_out, int64_t rows,
                int cols, float eps, float gamma_shift) {
  constexpr int N = Vec<T>::N;
  constexpr int RPB = BT / TPR;
  __shared__ float red[BT / 64];
  const int nvec = cols / N;
  const int lane = threadIdx.x % TPR;
  const int sub = threadIdx.x / TPR;
  const float inv_cols = 1.0f / (float)cols;

  Vec<T> g[VPT], b[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int v = lane + i * TPR;
    if (v < nvec) {
      g[i] = ldg(gamma + (int64_t)v * N);
      if (LN) b[i] = ldg(beta + (int64_t)v * N);
    }
  }

  for (int64_t row0 = (int64_t)blockIdx.x * RPB; row0 < rows; row0 += (int64_t)gridDim.x * RPB) {
    const int64_t row = row0 + sub;
    const bool active = row < rows;
    const T *xr = x + row * cols;
    Vec<T> xv[VPT];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int v = lane + i * TPR;
      if (active && v < nvec) {
        xv[i] = ldg_s<NT>(xr + (int64_t)v * N);
        if (RES) {
          // the row that is normalised is x + residual, rounded to the storage type and written out: what a
          // separate residual-add kernel in front of the norm would have stored and this one read back
          const Vec<T> rv = ldg_s<NT>(residual + row * cols + (int64_t)v * N);
#pragma unroll
          for (int j = 0; j < N; ++j) xv[i].v[j] = from_f<T>(to_f(xv[i].v[j]) + to_f(rv.v[j]));
          stg_s<NT>(sum_out + row * cols + (int64_t)v * N, xv[i]);
        }
#pragma unroll
        for (int j = 0; j < N; ++j) {
          const float f = to_f(xv[i].v[j]);
          s += LN ? f : f * f;
        }
      }
    }
    float mean = 0.f, var;
    if (LN) {
      s = (TPR == 64) ? wave_sum(s) : block_sum<BT>(s, red);
      mean = s * inv_cols;
      float s2 = 0.f;
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int v = lane + i * TPR;
        if (active && v < nvec) {
#pragma unroll
          for (int j = 0; j < N; ++j) {
            const float f = to_f(xv[i].v[j]) - mean;
            s2 += f * f;
          }
        }
      }
      s2 = (TPR == 64) ? wave_sum(s2) : block_sum<BT>(s2, red);
      var = s2 * inv_cols;
    } else {
      s = (TPR == 64) ? wave_sum(s) : block_sum<BT>(s, red);
      var = s * inv_cols;
    }
    const float rs = 1.0f / sqrtf(var + eps);
    if (active) {
      T *yr = y + row * cols;
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int v = lane + i * TPR;
        if (v < nvec) {
          Vec<T> o;
#pragma unroll
          for (int j = 0; j < N; ++j) {
            const float gm = to_f(g[i].v[j]) + gamma_shift;
            float f = (to_f(xv[i].v[j]) - mean) * rs * gm;
            if (LN) f += to_f(b[i].v[j]);
            o.v[j] = from_f<T>(f);
          }
          stg_s<NT>(yr + (int64_t)v * N, o);
        }
      }
      if (lane == 0) {
        rs_out[row] = rs;
        if (LN) mu_out[row] = mean;
      }
    }
  }
}

// Any cols / alignment: one block per row, scalar accesses, row re-read from cache.
template <typename T, bool LN>
__global__ void __launch_bounds__(256)
norm_fwd_generic_kernel(const T *__restrict__ x, const T *__restrict__ residual, T *__restrict__ sum_out,
                        const T *__restrict__ gamma, const T *__restrict__ beta,
                        T *__restrict__ y, float *__restrict__ mu_out, float *__restrict__ rs_out,
                        int64_t rows, int64_t cols, float eps, float gamma_shift) {
  __shared__ float red[4];
  const float inv_cols = 1.0f / (float)cols;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T *xr = x + row * cols;
    if (residual) {     // x + residual first, stored; every thread re-reads only the columns it wrote itself
      T *sr = sum_out + row * cols;
      for (int64_t c = threadIdx.x; c < cols; c += 256) sr[c] = from_f<T>(to_f(xr[c]) + to_f(residual[row * cols + c]));
      xr = sr;
    }
    float mean = 0.f;
    if (LN) {
      float s = 0.f;
      for (int64_t c = threadIdx.x; c < cols; c += 256) s += to_f(xr[c]);
      mean = block256_sum(s, red) * inv_cols;
    }
    float s2 = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += 256) {
      const float f = to_f(xr[c]) - mean;
      s2 += f * f;
    }
    const float rs = 1.0f / sqrtf(block256_sum(s2, red) * inv_cols + eps);
    T *yr = y + row * cols;
    for (int64_t c = threadIdx.x; c < cols; c += 256) {
      float f = (to_f(xr[c]) - mean) * rs * (to_f(gamma[c]) + gamma_shift);
      if (LN) f += to_f(beta[c]);
      yr[c] = from_f<T>(f);
    }
    if (threadIdx.x == 0) {
      rs_out[row] = rs;
      if (LN) mu_out[row] = mean;
    }
  }
}

// Backward main pass.  part: fp32 [2][gridDim.x][cols] (dgamma rows, then dbeta rows).
template <typename T, int BT, int TPR, int VPT, bool LN, bool NT, bool ADD>
__global__ void __launch_bounds__(BT)
norm_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ x, const float *__restrict__ mu,
                const float *__restrict__ rsigma, const T *__restrict__ gamma, const T *__restrict__ add_to_dx,
                T *__restrict__ dx, float *__restrict__ part, int64_t rows, int cols, float gamma_shift) {
  constexpr int N = Vec<T>::N;
  constexpr int RPB = BT / TPR;
  __shared__ float red[BT / 64];
  extern __shared__ float stage[];  // TPR==64 only: [4 waves][TPR*VPT*N] floats
  const int nvec = cols / N;
  const int lane = threadIdx.x % TPR;
  const int sub = threadIdx.x / TPR;
  const float inv_cols = 1.0f / (float)cols;

  Vec<T> g[VPT];
  float dg[VPT][N], db[VPT][N];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int v = lane + i * TPR;
    if (v < nvec) g[i] = ldg(gamma + (int64_t)v * N);
#pragma unroll
    for (int j = 0; j < N; ++j) {
      dg[i][j] = 0.f;
      db[i][j] = 0.f;
    }
  }

  // The next row's x and dy are requested before the current row's reduction, so that a block
  // keeps two rows of loads in flight.
  Vec<T> xn[VPT], dn[VPT];
  auto fetch = [&](int64_t row) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int v = lane + i * TPR;
      if (row < rows && v < nvec) {
        xn[i] = ldg_s<NT>(x + row * cols + (int64_t)v * N);
        dn[i] = ldg_s<NT>(dy + row * cols + (int64_t)v * N);
      }
    }
  };
  fetch((int64_t)blockIdx.x * RPB + sub);
  for (int64_t row0 = (int64_t)blockIdx.x * RPB; row0 < rows; row0 += (int64_t)gridDim.x * RPB) {
    const int64_t row = row0 + sub;
    const bool active = row < rows;
    Vec<T> xv[VPT], dv[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      xv[i] = xn[i];
      dv[i] = dn[i];
    }
    fetch(row + (int64_t)gridDim.x * RPB);
    Vec<T> rv[VPT];       // the gradient added to dx: requested ahead of the reduction
    if (ADD) {
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int v = lane + i * TPR;
        if (active && v < nvec) rv[i] = ldg_s<NT>(add_to_dx + row * cols + (int64_t)v * N);
      }
    }
    float rs = 0.f, mean = 0.f;
    if (active) {
      rs = rsigma[row];
      if (LN) mean = mu[row];
    }
    float s1 = 0.f, s2 = 0.f;  // sum g*xhat, sum g
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int v = lane + i * TPR;
      if (active && v < nvec) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
          const float xh = (to_f(xv[i].v[j]) - mean) * rs;
          const float d = to_f(dv[i].v[j]);
          const float gg = d * (to_f(g[i].v[j]) + gamma_shift);
          s1 += gg * xh;
          if (LN) s2 += gg;
          dg[i][j] += d * xh;
          if (LN) db[i][j] += d;
        }
      }
    }
    if (TPR == 64) {
      s1 = wave_sum(s1);
      if (LN) s2 = wave_sum(s2);
    } else {
      s1 = block_sum<BT>(s1, red);
      if (LN) s2 = block_sum<BT>(s2, red);
    }
    const float c1 = s1 * inv_cols, c2 = s2 * inv_cols;
    if (active) {
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int v = lane + i * TPR;
        if (v < nvec) {
          Vec<T> o;
#pragma unroll
          for (int j = 0; j < N; ++j) {
            const float xh = (to_f(xv[i].v[j]) - mean) * rs;
            const float gg = to_f(dv[i].v[j]) * (to_f(g[i].v[j]) + gamma_shift);
            float f = rs * (gg - xh * c1 - c2);
            if (ADD) f += to_f(rv[i].v[j]);
            o.v[j] = from_f<T>(f);
          }
          stg_s<NT>(dx + row * cols + (int64_t)v * N, o);
        }
      }
    }
  }

  // Per-block partial dgamma/dbeta.  With one wave per row the four waves own
  // the same columns: stage through LDS and add in wave order.
  float *pg = part + (int64_t)blockIdx.x * cols;
  float *pb = part + ((int64_t)gridDim.x + blockIdx.x) * cols;
  if (TPR == 64) {
    constexpr int W = 64 * VPT * N;  // staged columns per wave
#pragma unroll
    for (int pass = 0; pass < (LN ? 2 : 1); ++pass) {
      __syncthreads();
#pragma unroll
      for (int i = 0; i < VPT; ++i)
#pragma unroll
        for (int j = 0; j < N; ++j)
          stage[sub * W + (i * 64 + lane) * N + j] = pass == 0 ? dg[i][j] : db[i][j];
      __syncthreads();
      float *dst = pass == 0 ? pg : pb;
      for (int c = threadIdx.x; c < W; c += 256) {
        // staged column c corresponds to vector (c / N) = i*64 + lane, element c % N
        const int v = c / N;
        if (v < nvec) {
          const float t = (stage[c] + stage[W + c]) + (stage[2 * W + c] + stage[3 * W + c]);
          dst[(int64_t)v * N + (c % N)] = t;
        }
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int v = lane + i * TPR;
      if (v < nvec) {
#pragma unroll
        for (int j = 0; j < N; j += 4) {
          *reinterpret_cast<float4 *>(pg + (int64_t)v * N + j) =
              make_float4(dg[i][j], dg[i][j + 1], dg[i][j + 2], dg[i][j + 3]);
          if (LN)
            *reinterpret_cast<float4 *>(pb + (int64_t)v * N + j) =
                make_float4(db[i][j], db[i][j + 1], db[i][j + 2], db[i][j + 3]);
        }
      }
    }
  }
}

template <typename T, bool LN>
__global__ void __launch_bounds__(256)
norm_bwd_generic_kernel(const T *__restrict__ dy, const T *__restrict__ x, const float *__restrict__ mu,
                        const float *__restrict__ rsigma, const T *__restrict__ gamma,
                        const T *__restrict__ add_to_dx, T *__restrict__ dx, int64_t rows, int64_t cols,
                        float gamma_shift) {
  __shared__ float red[4];
  const float inv_cols = 1.0f / (float)cols;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const float rs = rsigma[row];
    const float mean = LN ? mu[row] : 0.f;
    float s1 = 0.f, s2 = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += 256) {
      const float xh = (to_f(x[row * cols + c]) - mean) * rs;
      const float gg = to_f(dy[row * cols + c]) * (to_f(gamma[c]) + gamma_shift);
      s1 += gg * xh;
      s2 += gg;
    }
    const float c1 = block256_sum(s1, red) * inv_cols;
    const float c2 = LN ? block256_sum(s2, red) * inv_cols : 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += 256) {
      const float xh = (to_f(x[row * cols + c]) - mean) * rs;
      const float gg = to_f(dy[row * cols + c]) * (to_f(gamma[c]) + gamma_shift);
      float f = rs * (gg - xh * c1 - c2);
      if (add_to_dx) f += to_f(add_to_dx[row * cols + c]);
      dx[row * cols + c] = from_f<T>(f);
    }
  }
}

// Column sums for the generic path: part [2][nchunks][cols]; block (bx, by)
// handles 64 columns x one chunk of rows.
template <typename T, bool LN>
__global__ void __launch_bounds__(256)
norm_bwd_generic_wgrad_kernel(const T *__restrict__ dy, const T *__restrict__ x, const float *__restrict__ mu,
                              const float *__restrict__ rsigma, float *__restrict__ part, int64_t rows,
                              int64_t cols, int64_t rows_per_chunk) {
  __shared__ float sg[4][64], sb[4][64];
  const int cx = threadIdx.x & 63, ry = threadIdx.x >> 6;
  const int64_t c = (int64_t)blockIdx.x * 64 + cx;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < rows ? r0 + rows_per_chunk : rows;
  float ag = 0.f, ab = 0.f;
  if (c < cols) {
    for (int64_t r = r0 + ry; r < r1; r += 4) {
      const float d = to_f(dy[r * cols + c]);
      const float xh = (to_f(x[r * cols + c]) - (LN ? mu[r] : 0.f)) * rsigma[r];
      ag += d * xh;
      ab += d;
    }
  }
  sg[ry][cx] = ag;
  sb[ry][cx] = ab;
  __syncthreads();
  if (ry == 0 && c < cols) {
    part[(int64_t)blockIdx.y * cols + c] = (sg[0][cx] + sg[1][cx]) + (sg[2][cx] + sg[3][cx]);
    if (LN) part[((int64_t)gridDim.y + blockIdx.y) * cols + c] = (sb[0][cx] + sb[1][cx]) + (sb[2][cx] + sb[3][cx]);
  }
}

// Backward in ONE launch for inputs that stay in the caches (a few hundred rows): no partial rows, no finalize.
// dx needs a whole row (its two row sums), the weight gradients need a whole column:
//     dgamma[c] = sum_r dy[r][c] * (x[r][c] - mu[r]) * rsigma[r],    dbeta[c] = sum_r dy[r][c],
// and mu / rsigma are inputs (saved by the forward), so a column sum depends on no other workgroup.  Workgroup w
// therefore does both: the rows w, w + G, ... for dx exactly as norm_bwd_kernel does (same arithmetic, same bits),
// and the column slab [SW w, SW w + SW) over ALL rows for dgamma / dbeta, reading that slab a second time (from
// L2 / the last-level cache: the operands were just streamed through it).  Row groups of the slab are added
// through LDS in a fixed order.  1024 threads, one 16-byte vector of the row per thread (cols <= 1024 vectors).
template <typename T, bool LN, bool ADD>
__global__ void __launch_bounds__(1024)
norm_bwd_onepass_kernel(const T *__restrict__ dy, const T *__restrict__ x, const float *__restrict__ mu,
                        const float *__restrict__ rsigma, const T *__restrict__ gamma, const T *__restrict__ add_to_dx,
                        T *__restrict__ dx, T *__restrict__ dgamma, T *__restrict__ dbeta, int64_t rows, int cols,
                        float gamma_shift, int accumulate) {
  constexpr int N = Vec<T>::N;
  constexpr int BT = 1024;
  constexpr int SW = 32;                 // columns of a slab
  constexpr int L = SW / N;              // lanes across a slab row
  constexpr int RG = BT / L;             // row groups of the column phase
  constexpr int PRE = 2;                 // slab iterations requested before the row phase
  __shared__ float red[BT / 64];
  __shared__ float sg[RG][SW + 1];
  __shared__ float sb[LN ? RG : 1][SW + 1];
  const int nvec = cols / N;
  const int tid = threadIdx.x;
  const float inv_cols = 1.0f / (float)cols;

  // ---- column phase, part 1: the first PRE row groups' loads go out now ----
  const int cl = tid % L, rg = tid / L;
  const int cv = (int)blockIdx.x * L + cl;             // vector index inside a row
  const bool cvalid = cv < nvec;
  Vec<T> sx[PRE], sd[PRE];
  float srs[PRE], smu[PRE];
#pragma unroll
  for (int u = 0; u < PRE; ++u) {
    const int64_t r = rg + (int64_t)u * RG;
    srs[u] = 0.f;
    smu[u] = 0.f;
    if (cvalid && r < rows) {
      sx[u] = ldg(x + r * cols + (int64_t)cv * N);
      sd[u] = ldg(dy + r * cols + (int64_t)cv * N);
      srs[u] = rsigma[r];
      if (LN) smu[u] = mu[r];
    }
  }

  // ---- row phase: dx of rows blockIdx.x, blockIdx.x + gridDim.x, ... ----
  {
    const int v = tid;
    const bool vvalid = v < nvec;
    Vec<T> g;
    if (vvalid) g = ldg(gamma + (int64_t)v * N);
    Vec<T> xn, dn;
    auto fetch = [&](int64_t row) {
      if (row < rows && vvalid) {
        xn = ldg(x + row * cols + (int64_t)v * N);
        dn = ldg(dy + row * cols + (int64_t)v * N);
      }
    };
    fetch(blockIdx.x);
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
      const Vec<T> xv = xn, dv = dn;
      fetch(row + gridDim.x);
      Vec<T> rv;
      if (ADD && vvalid) rv = ldg(add_to_dx + row * cols + (int64_t)v * N);
      const float rs = rsigma[row];
      const float mean = LN ? mu[row] : 0.f;
      float s1 = 0.f, s2 = 0.f;
      if (vvalid) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
          const float xh = (to_f(xv.v[j]) - mean) * rs;
          const float gg = to_f(dv.v[j]) * (to_f(g.v[j]) + gamma_shift);
          s1 += gg * xh;
          if (LN) s2 += gg;
        }
      }
      s1 = block_sum<BT>(s1, red);
      if (LN) s2 = block_sum<BT>(s2, red);
      const float c1 = s1 * inv_cols, c2 = s2 * inv_cols;
      if (vvalid) {
        Vec<T> o;
#pragma unroll
        for (int j = 0; j < N; ++j) {
          const float xh = (to_f(xv.v[j]) - mean) * rs;
          const float gg = to_f(dv.v[j]) * (to_f(g.v[j]) + gamma_shift);
          float f = rs * (gg - xh * c1 - c2);
          if (ADD) f += to_f(rv.v[j]);
          o.v[j] = from_f<T>(f);
        }
        stg(dx + row * cols + (int64_t)v * N, o);
      }
    }
  }

  // ---- column phase, part 2: accumulate the slab over all rows, row groups in order ----
  float dg[N], db[N];
#pragma unroll
  for (int j = 0; j < N; ++j) {
    dg[j] = 0.f;
    db[j] = 0.f;
  }
#pragma unroll
  for (int u = 0; u < PRE; ++u) {
    const int64_t r = rg + (int64_t)u * RG;
    if (cvalid && r < rows) {
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const float d = to_f(sd[u].v[j]);
        dg[j] += d * ((to_f(sx[u].v[j]) - smu[u]) * srs[u]);
        if (LN) db[j] += d;
      }
    }
  }
  if (cvalid) {
    for (int64_t r = rg + (int64_t)PRE * RG; r < rows; r += RG) {
      const Vec<T> xv = ldg(x + r * cols + (int64_t)cv * N), dv = ldg(dy + r * cols + (int64_t)cv * N);
      const float rs = rsigma[r];
      const float mean = LN ? mu[r] : 0.f;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const float d = to_f(dv.v[j]);
        dg[j] += d * ((to_f(xv.v[j]) - mean) * rs);
        if (LN) db[j] += d;
      }
    }
  }
#pragma unroll
  for (int j = 0; j < N; ++j) {
    sg[rg][cl * N + j] = dg[j];
    if (LN) sb[rg][cl * N + j] = db[j];
  }
  __syncthreads();
  // column c: 32 threads add RG / 32 row groups each (k, k + 32, ...), then thread k = 0 adds the 32 sums in order
  {
    const int c = tid / 32, k = tid % 32;
    float ag = 0.f, ab = 0.f;
#pragma unroll
    for (int r = k; r < RG; r += 32) {
      ag += sg[r][c];
      if (LN) ab += sb[r][c];
    }
    __syncthreads();
    sg[k][c] = ag;
    if (LN) sb[k][c] = ab;
    __syncthreads();
    const int64_t col = (int64_t)blockIdx.x * SW + c;
    if (k == 0 && col < cols) {
      float tg = 0.f, tb = 0.f;
#pragma unroll
      for (int r = 0; r < 32; ++r) {
        tg += sg[r][c];
        if (LN) tb += sb[r][c];
      }
      if (accumulate) {
        tg += to_f(dgamma[col]);
        if (LN) tb += to_f(dbeta[col]);
      }
      dgamma[col] = from_f<T>(tg);
      if (LN) dbeta[col] = from_f<T>(tb);
    }
  }
}

// Reduce partial rows: part [2][P][cols] -> dgamma (and dbeta) [cols].
// Block = 16 float4 lanes (64 columns) x 16 row groups; each lane streams its rows with four
// independent accumulators, the row groups are combined through LDS in a fixed order.
template <typename T, bool LN>
__global__ void __launch_bounds__(256)
norm_bwd_finalize_kernel(const float *__restrict__ part, T *__restrict__ dgamma, T *__restrict__ dbeta, int P,
                         int64_t cols, int accumulate) {
  __shared__ float4 sg[16][16], sb[16][16];
  const int cx = threadIdx.x & 15, ry = threadIdx.x >> 4;
  const int64_t c = (int64_t)blockIdx.x * 64 + cx * 4;
  float4 ag[4], ab[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    ag[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    ab[u] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  if (c < cols) {   // cols is a multiple of 4 on this path
    for (int p0 = ry; p0 < P; p0 += 64) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int p = p0 + 16 * u;
        if (p < P) {
          const float4 v = *reinterpret_cast<const float4 *>(part + (int64_t)p * cols + c);
          ag[u].x += v.x; ag[u].y += v.y; ag[u].z += v.z; ag[u].w += v.w;
          if (LN) {
            const float4 w = *reinterpret_cast<const float4 *>(part + ((int64_t)P + p) * cols + c);
            ab[u].x += w.x; ab[u].y += w.y; ab[u].z += w.z; ab[u].w += w.w;
          }
        }
      }
    }
  }
  auto fold = [](const float4 (&a)[4]) {
    return make_float4((a[0].x + a[1].x) + (a[2].x + a[3].x), (a[0].y + a[1].y) + (a[2].y + a[3].y),
                       (a[0].z + a[1].z) + (a[2].z + a[3].z), (a[0].w + a[1].w) + (a[2].w + a[3].w));
  };
  sg[ry][cx] = fold(ag);
  sb[ry][cx] = fold(ab);
  __syncthreads();
  if (ry == 0 && c < cols) {
    float tg[4] = {0.f, 0.f, 0.f, 0.f}, tb[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      tg[0] += sg[r][cx].x; tg[1] += sg[r][cx].y; tg[2] += sg[r][cx].z; tg[3] += sg[r][cx].w;
      tb[0] += sb[r][cx].x; tb[1] += sb[r][cx].y; tb[2] += sb[r][cx].z; tb[3] += sb[r][cx].w;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (accumulate) {
        tg[e] += to_f(dgamma[c + e]);
        if (LN) tb[e] += to_f(dbeta[c + e]);
      }
      dgamma[c + e] = from_f<T>(tg[e]);
      if (LN) dbeta[c + e] = from_f<T>(tb[e]);
    }
  }
}

// Same reduction for column counts that are not a multiple of 4 (generic path).
template <typename T, bool LN>
__global__ void __launch_bounds__(256)
norm_bwd_finalize_scalar_kernel(const float *__restrict__ part, T *__restrict__ dgamma, T *__restrict__ dbeta, int P,
                                int64_t cols, int accumulate) {
  __shared__ float sg[8][33], sb[8][33];
  const int cx = threadIdx.x & 31, ry = threadIdx.x >> 5;
  const int64_t c = (int64_t)blockIdx.x * 32 + cx;
  float ag = 0.f, ab = 0.f;
  if (c < cols) {
    for (int p = ry; p < P; p += 8) {
      ag += part[(int64_t)p * cols + c];
      if (LN) ab += part[((int64_t)P + p) * cols + c];
    }
  }
  sg[ry][cx] = ag;
  sb[ry][cx] = ab;
  __syncthreads();
  if (ry == 0 && c < cols) {
    float tg = 0.f, tb = 0.f;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      tg += sg[r][cx];
      tb += sb[r][cx];
    }
    if (accumulate) {
      tg += to_f(dgamma[c]);
      if (LN) tb += to_f(dbeta[c]);
    }
    dgamma[c] = from_f<T>(tg);
    if (LN) dbeta[c] = from_f<T>(tb);
  }
}

// ---- host side --------------------------------------------------------------------
struct NormPlan {
  bool vec;   // vector path usable
  int tpr;    // threads per row (64: one wave per row, 4 rows per 256-thread block; 256; 1024)
  int vpt;    // 16-byte vectors per thread
};

// Wide rows are spread over 1024 threads so that a thread keeps few columns: the backward's
// per-column accumulators then fit in few registers and many waves stay resident.
static NormPlan norm_plan(int64_t cols, int elt, bool all_aligned) {
  NormPlan p{false, 0, 0};
  const int n = 16 / elt;
  if (!all_aligned || cols % n != 0 || cols <= 0) return p;
  const int64_t nvec = cols / n;
  if (nvec <= 64 * 4) {
    p.tpr = 64;
    p.vpt = nvec <= 64 ? 1 : (nvec <= 128 ? 2 : 4);
  } else if (nvec <= 512) {
    p.tpr = 256;
    p.vpt = 2;
  } else if (nvec <= 2048) {
    p.tpr = 1024;
    p.vpt = nvec <= 1024 ? 1 : 2;
  } else {
    return p;
  }
  p.vec = true;
  return p;
}

static int64_t bwd_blocks(int64_t rows, int64_t cols, int elt) {
  const NormPlan p = norm_plan(cols, elt, true);
  if (!p.vec) {
    // generic path: number of row chunks for the column-sum kernel
    int64_t chunks = cdiv(rows, 64);
    return chunks < 1 ? 1 : (chunks > 256 ? 256 : chunks);
  }
  const int rpb = p.tpr == 64 ? 4 : 1;
  const int64_t iters = cdiv(rows, rpb);
  // Every block leaves one fp32 partial row per weight gradient, written once and read once by the
  // finalize kernel: with one block per row that traffic exceeds the operands' own for a few hundred
  // rows.  256 blocks already keep the memory system full (measured: 512 -> 256 partial rows takes the
  // 512-row case from 21 to 16 us and 4096 rows from 47 to 39 us, 32768 rows unchanged); below 32 MB of
  // operand traffic 128 are better still (14 us at 512 rows).
  const int64_t cap = 3 * rows * cols * elt < (32ll << 20) ? 128 : 256;
  int64_t nb = iters;
  if (nb > cap) nb = cap;
  if (nb < 1) nb = 1;
  return nb;
}

// Whether the backward runs as one launch (norm_bwd_onepass_kernel): rows of 513 .. 1024 vectors (one vector per
// thread of a 1024-thread workgroup) and operands small enough that the second, column-wise read of dy and x is
// served by the caches (32 MiB of dy + x; the 512 x 8192 16-bit rows of a sequence-parallel shard are 16 MiB).
static bool bwd_onepass(const NormPlan &p, int64_t rows, int64_t cols, int elt) {
  return p.vec && p.tpr == 1024 && p.vpt == 1 && rows > 0 && 2 * rows * cols * elt <= (32ll << 20);
}

template <typename T, bool LN>
static int launch_fwd(const NormPlan &p, const T *x, const T *residual, T *sum_out, const T *gamma, const T *beta, T *y,
                      float *mu, float *rs, int64_t rows, int64_t cols, float eps, float shift, hipStream_t st) {
  if (!p.vec) {
    int64_t nb = rows < 4096 ? rows : 4096;
    hipLaunchKernelGGL((norm_fwd_generic_kernel<T, LN>), dim3((unsigned)nb), dim3(256), 0, st, x, residual, sum_out,
                       gamma, beta, y, mu, rs, rows, cols, eps, shift);
    return 0;
  }
  const int rpb = p.tpr == 64 ? 4 : 1;
  int64_t nb = cdiv(rows, rpb);
  if (nb > 256 * 16) nb = 256 * 16;
  const bool nt = stream_hint((residual ? 4 : 2) * rows * cols * (int64_t)sizeof(T));
#define L3(BT, TPR, VPT, NT, RES)                                                                            \
  hipLaunchKernelGGL((norm_fwd_kernel<T, BT, TPR, VPT, LN, NT, RES>), dim3((unsigned)nb), dim3(BT), 0, st, x,     \
                     residual, sum_out, gamma, beta, y, mu, rs, rows, (int)cols, eps, shift)
#define L2(BT, TPR, VPT, NT)                                                                                 \
  do {                                                                                                       \
    if (residual) L3(BT, TPR, VPT, NT, true); else L3(BT, TPR, VPT, NT, false);                               \
  } while (0)
#define L(BT, TPR, VPT)                                                                                      \
  do {                                                                                                       \
    if (nt) L2(BT, TPR, VPT, true); else L2(BT, TPR, VPT, false);                                             \
  } while (0)
  if (p.tpr == 64) {
    if (p.vpt == 1) L(256, 64, 1); else if (p.vpt == 2) L(256, 64, 2); else L(256, 64, 4);
  } else if (p.tpr == 256) {
    L(256, 256, 2);
  } else {
    // From 2048 rows of up to 1024 vectors the forward runs four vectors per thread in 256-thread blocks: eight rows
    // per compute unit in flight instead of two (rows of 8192 bf16: 24.1 against 26.6 us at 4096 rows, 13.8 against
    // 15.2 us at 2048, level from 8192 rows on; rows of 5120: 17.2 against 21.7 us).  Fewer rows, and wider ones
    // (eight vectors per thread), are faster in the 1024-thread form.  The choice does not look at the residual
    // operand (with it the two forms are within 3 % of each other), so that the fused add + norm sums a row in the
    // same order as the norm alone and the two give the same bits.
    if (rows >= 2048 && cols / (16 / (int64_t)sizeof(T)) <= 1024) {
      L(256, 256, 4);
    } else {
      if (p.vpt == 1) L(1024, 1024, 1); else L(1024, 1024, 2);
    }
  }
#undef L
#undef L2
#undef L3
  return 0;
}

template <typename T, bool LN>
static int launch_bwd(const NormPlan &p, const T *dy, const T *x, const float *mu, const float *rs, const T *gamma,
                      const T *add, T *dx, T *dgamma, T *dbeta, float *part, int64_t rows, int64_t cols,
                      float shift, int accumulate, hipStream_t st) {
  const int64_t nb = bwd_blocks(rows, cols, sizeof(T));
  if (bwd_onepass(p, rows, cols, sizeof(T))) {
    const unsigned g = (unsigned)cdiv(cols, 32);
    if (add)
      hipLaunchKernelGGL((norm_bwd_onepass_kernel<T, LN, true>), dim3(g), dim3(1024), 0, st, dy, x, mu, rs, gamma, add,
                         dx, dgamma, dbeta, rows, (int)cols, shift, accumulate);
    else
      hipLaunchKernelGGL((norm_bwd_onepass_kernel<T, LN, false>), dim3(g), dim3(1024), 0, st, dy, x, mu, rs, gamma, add,
                         dx, dgamma, dbeta, rows, (int)cols, shift, accumulate);
    return 0;
  }
  if (!p.vec) {
    int64_t g = rows < 4096 ? rows : 4096;
    hipLaunchKernelGGL((norm_bwd_generic_kernel<T, LN>), dim3((unsigned)g), dim3(256), 0, st, dy, x, mu, rs, gamma,
                       add, dx, rows, cols, shift);
    const int64_t rpc = cdiv(rows, nb);
    hipLaunchKernelGGL((norm_bwd_generic_wgrad_kernel<T, LN>), dim3((unsigned)cdiv(cols, 64), (unsigned)nb),
                       dim3(256), 0, st, dy, x, mu, rs, part, rows, cols, rpc);
  } else {
    const bool nt = stream_hint((add ? 4 : 3) * rows * cols * (int64_t)sizeof(T));
#define L3(BT, TPR, VPT, NT, ADD)                                                                            \
  hipLaunchKernelGGL((norm_bwd_kernel<T, BT, TPR, VPT, LN, NT, ADD>), dim3((unsigned)nb), dim3(BT),               \
                     (TPR == 64 ? 4 * 64 * VPT * (16 / sizeof(T)) * sizeof(float) : 0), st, dy, x, mu, rs, gamma, \
                     add, dx, part, rows, (int)cols, shift)
#define L2(BT, TPR, VPT, NT)                                                                                 \
  do {                                                                                                       \
    if (add) L3(BT, TPR, VPT, NT, true); else L3(BT, TPR, VPT, NT, false);                                    \
  } while (0)
#define L(BT, TPR, VPT)                                                                                      \
  do {                                                                                                       \
    if (nt) L2(BT, TPR, VPT, true); else L2(BT, TPR, VPT, false);                                             \
  } while (0)
    if (p.tpr == 64) {
      if (p.vpt == 1) L(256, 64, 1); else if (p.vpt == 2) L(256, 64, 2); else L(256, 64, 4);
    } else if (p.tpr == 256) {
      L(256, 256, 2);
    } else {
      if (p.vpt == 1) L(1024, 1024, 1); else L(1024, 1024, 2);
    }
#undef L
#undef L2
#undef L3
  }
  if (cols % 4 == 0)
    hipLaunchKernelGGL((norm_bwd_finalize_kernel<T, LN>), dim3((unsigned)cdiv(cols, 64)), dim3(256), 0, st, part,
                       dgamma, dbeta, (int)nb, cols, accumulate);
  else
    hipLaunchKernelGGL((norm_bwd_finalize_scalar_kernel<T, LN>), dim3((unsigned)cdiv(cols, 32)), dim3(256), 0, st,
                       part, dgamma, dbeta, (int)nb, cols, accumulate);
  return 0;
}

}  // namespace dh

static int norm_fwd_entry(const void *x, const void *residual, void *sum_out, const void *gamma, const void *beta,
                          void *y, float *mu, float *rsigma, int64_t rows, int64_t cols, float eps,
                          int zero_centered_gamma, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(rows >= 0 && cols > 0, "bad shape rows=%lld cols=%lld", (long long)rows, (long long)cols);
  if (rows == 0) return DH_OK;
  DH_CHECK(x && gamma && y && rsigma, "null pointer");
  DH_CHECK((residual == nullptr) == (sum_out == nullptr), "residual and sum_out go together");
  DH_CHECK(beta == nullptr || mu != nullptr, "LayerNorm (beta given) needs a mu output");
  DH_CHECK(cols < (1ll << 31), "cols too large");
  const bool al = aligned16(x) && aligned16(y) && aligned16(gamma) && (beta == nullptr || aligned16(beta)) &&
                  (residual == nullptr || (aligned16(residual) && aligned16(sum_out)));
  const float shift = zero_centered_gamma ? 1.0f : 0.0f;
  hipStream_t st = (hipStream_t)stream;
  DH_DISPATCH_DTYPE(dtype, {
    const NormPlan p = norm_plan(cols, sizeof(T), al);
    if (beta)
      launch_fwd<T, true>(p, (const T *)x, (const T *)residual, (T *)sum_out, (const T *)gamma, (const T *)beta, (T *)y,
                          mu, rsigma, rows, cols, eps, shift, st);
    else
      launch_fwd<T, false>(p, (const T *)x, (const T *)residual, (T *)sum_out, (const T *)gamma, nullptr, (T *)y, mu,
                           rsigma, rows, cols, eps, shift, st);
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

extern "C" int dh_norm_fwd(const void *x, const void *gamma, const void *beta, void *y, float *mu, float *rsigma,
                           int64_t rows, int64_t cols, float eps, int zero_centered_gamma, int dtype,
                           void *stream) {
  return norm_fwd_entry(x, nullptr, nullptr, gamma, beta, y, mu, rsigma, rows, cols, eps, zero_centered_gamma, dtype,
                        stream);
}

extern "C" int dh_add_norm_fwd(const void *x, const void *residual, void *sum_out, const void *gamma, const void *beta,
                               void *y, float *mu, float *rsigma, int64_t rows, int64_t cols, float eps,
                               int zero_centered_gamma, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(rows <= 0 || (residual && sum_out), "null pointer");
  return norm_fwd_entry(x, residual, sum_out, gamma, beta, y, mu, rsigma, rows, cols, eps, zero_centered_gamma, dtype,
                        stream);
}

extern "C" size_t dh_norm_bwd_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 16;
  // The block count depends on the element size only through the vector-path
  // test; take the larger of the two cases.
  const int64_t a = dh::bwd_blocks(rows, cols, 2), b = dh::bwd_blocks(rows, cols, 4);
  return (size_t)(2 * (a > b ? a : b) * cols * (int64_t)sizeof(float));
}

namespace dh {
__global__ void __launch_bounds__(256) zero_bytes_kernel(uint8_t *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) p[i] = 0;
}
}  // namespace dh

extern "C" int dh_norm_bwd(const void *dy, const void *x, const float *mu, const float *rsigma, const void *gamma,
                           const void *add_to_dx, void *dx, void *dgamma, void *dbeta, void *workspace,
                           size_t workspace_bytes, int64_t rows, int64_t cols, int zero_centered_gamma,
                           int accumulate_wgrad, int dtype, void *stream) {
  using namespace dh;
  DH_CHECK(rows >= 0 && cols > 0, "bad shape rows=%lld cols=%lld", (long long)rows, (long long)cols);
  DH_CHECK(dy && x && rsigma && gamma && dx && dgamma && workspace, "null pointer");
  DH_CHECK(workspace_bytes >= dh_norm_bwd_workspace_bytes(rows, cols),
           "workspace of %zu bytes is smaller than dh_norm_bwd_workspace_bytes(%lld, %lld) = %zu", workspace_bytes,
           (long long)rows, (long long)cols, dh_norm_bwd_workspace_bytes(rows, cols));
  DH_CHECK(mu == nullptr || dbeta != nullptr, "LayerNorm backward (mu given) needs a dbeta output");
  DH_CHECK(cols < (1ll << 31), "cols too large");
  DH_CHECK(aligned16(workspace), "workspace must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (rows == 0) {
    // no rows: the weight gradients are zero (or unchanged when accumulating)
    // (a fill kernel, not a memset: memset nodes are unreliable inside a captured graph)
    if (!accumulate_wgrad) {
      const int64_t nbytes = cols * (int64_t)dtype_size(dtype);
      const unsigned blocks = (unsigned)(cdiv(nbytes, 256) < 1024 ? cdiv(nbytes, 256) : 1024);
      hipLaunchKernelGGL(zero_bytes_kernel, dim3(blocks), dim3(256), 0, st, (uint8_t *)dgamma, nbytes);
      if (mu && dbeta) hipLaunchKernelGGL(zero_bytes_kernel, dim3(blocks), dim3(256), 0, st, (uint8_t *)dbeta, nbytes);
      DH_LAUNCH_CHECK();
    }
    return DH_OK;
  }
  const bool al = aligned16(x) && aligned16(dy) && aligned16(dx) && aligned16(gamma) &&
                  (add_to_dx == nullptr || aligned16(add_to_dx));
  const float shift = zero_centered_gamma ? 1.0f : 0.0f;
  DH_DISPATCH_DTYPE(dtype, {
    NormPlan p = norm_plan(cols, sizeof(T), al);
    if (mu)
      launch_bwd<T, true>(p, (const T *)dy, (const T *)x, mu, rsigma, (const T *)gamma, (const T *)add_to_dx,
                          (T *)dx, (T *)dgamma, (T *)dbeta, (float *)workspace, rows, cols, shift,
                          accumulate_wgrad, st);
    else
      launch_bwd<T, false>(p, (const T *)dy, (const T *)x, nullptr, rsigma, (const T *)gamma,
                           (const T *)add_to_dx, (T *)dx, (T *)dgamma, nullptr, (float *)workspace, rows, cols,
                           shift, accumulate_wgrad, st);
  });
  DH_LAUNCH_CHECK();
  return DH_OK;
}

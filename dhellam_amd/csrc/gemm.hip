// Dense GEMM entry point: the reference's cuBLASLt call (csrc/operators/gemm.cu:3-170) made with hipBLASLt.
// Host code only: plain dense products are library work on this path; the hand-written matrix kernels of
// this library are the attention and grouped-GEMM ones.
//
// Convention of the reference, kept as is: A, B and D are row-major arrays handed to a column-major
// library, so with
//     m = transa ? a_rows : a_cols,   k = transa ? a_cols : a_rows,   n = transb ? b_cols : b_rows
// the result is the row-major D [n, m]:
//     transa  transb   D
//     1       0        B   @ A^T     ("TN": activations times weight^T)
//     0       0        B   @ A       ("NN": data gradient)
//     0       1        B^T @ A       ("NT": weight gradient)
#include <hipblaslt/hipblaslt.h>

#include <mutex>
#include <unordered_map>

#include "common.h"
#include "dhellam_hip.h"

namespace {

#define DH_BLAS(call)                                                                              \
  do {                                                                                             \
    hipblasStatus_t s_ = (call);                                                                   \
    if (s_ != HIPBLAS_STATUS_SUCCESS) {                                                            \
      ::dh::set_error(__FILE__, __LINE__, __func__, "hipBLASLt error %d in %s", (int)s_, #call);   \
      return DH_ERR_HIP;                                                                           \
    }                                                                                              \
  } while (0)

struct Key {
  int64_t m, n, k;
  size_t ws;
  int dev, flags;   // transa | transb << 1 | accumulate << 2 | dtype << 3 | out_dtype << 6
  bool operator==(const Key &o) const {
    return m == o.m && n == o.n && k == o.k && ws == o.ws && dev == o.dev && flags == o.flags;
  }
};
struct KeyHash {
  size_t operator()(const Key &x) const {
    size_t h = 1469598103934665603ull;
    for (uint64_t v : {(uint64_t)x.m, (uint64_t)x.n, (uint64_t)x.k, (uint64_t)x.ws, (uint64_t)x.dev, (uint64_t)x.flags})
      h = (h ^ v) * 1099511628211ull;
    return h;
  }
};

// One problem description per (shape, layout, types, device): built once, reused by every later call.
struct Plan {
  hipblasLtMatmulDesc_t op = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t ws_needed = 0;
};

std::mutex g_mu;
hipblasLtHandle_t g_handle[64] = {};
std::unordered_map<Key, Plan, KeyHash> g_plans;

hipDataType blas_type(int dtype) { return dtype == DH_BF16 ? HIP_R_16BF : dtype == DH_F16 ? HIP_R_16F : HIP_R_32F; }

int make_plan(hipblasLtHandle_t h, const Key &key, int transa, int transb, int dtype, int out_dtype, Plan &pl) {
  const int64_t m = key.m, n = key.n, k = key.k;
  const int64_t lda = transa ? k : m, ldb = transb ? n : k, ldd = m;
  DH_BLAS(hipblasLtMatrixLayoutCreate(&pl.a, blas_type(dtype), transa ? k : m, transa ? m : k, lda));
  DH_BLAS(hipblasLtMatrixLayoutCreate(&pl.b, blas_type(dtype), transb ? n : k, transb ? k : n, ldb));
  DH_BLAS(hipblasLtMatrixLayoutCreate(&pl.d, blas_type(out_dtype), m, n, ldd));
  DH_BLAS(hipblasLtMatmulDescCreate(&pl.op, HIPBLAS_COMPUTE_32F, HIP_R_32F));
  const hipblasOperation_t ta = transa ? HIPBLAS_OP_T : HIPBLAS_OP_N, tb = transb ? HIPBLAS_OP_T : HIPBLAS_OP_N;
  DH_BLAS(hipblasLtMatmulDescSetAttribute(pl.op, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)));
  DH_BLAS(hipblasLtMatmulDescSetAttribute(pl.op, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)));
  hipblasLtMatmulPreference_t pref = nullptr;
  DH_BLAS(hipblasLtMatmulPreferenceCreate(&pref));
  const uint64_t ws = key.ws;
  hipblasStatus_t s = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
  hipblasLtMatmulHeuristicResult_t res[1];
  int found = 0;
  if (s == HIPBLAS_STATUS_SUCCESS)
    s = hipblasLtMatmulAlgoGetHeuristic(h, pl.op, pl.a, pl.b, pl.d, pl.d, pref, 1, res, &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS || found < 1) {
    ::dh::set_error(__FILE__, __LINE__, __func__, "hipBLASLt has no kernel for m=%lld n=%lld k=%lld (status %d)",
                    (long long)m, (long long)n, (long long)k, (int)s);
    return DH_ERR_UNSUPPORTED;
  }
  pl.algo = res[0].algo;
  pl.ws_needed = res[0].workspaceSize;
  return DH_OK;
}

}  // namespace

static int gemm_entry(const void *a, const void *b, void *d, int64_t a_rows, int64_t a_cols, int64_t b_rows,
                      int64_t b_cols, int transa, int transb, int accumulate, int dtype, int out_dtype,
                      void *workspace, size_t workspace_bytes, void *stream) {
  DH_CHECK(dtype == DH_BF16 || dtype == DH_F16 || dtype == DH_F32, "unknown dtype %d", dtype);
  DH_CHECK(out_dtype == dtype || out_dtype == DH_F32, "the result is of the operands' type or fp32");
  DH_CHECK(a_rows >= 0 && a_cols >= 0 && b_rows >= 0 && b_cols >= 0, "negative size");
  const int64_t m = transa ? a_rows : a_cols, k = transa ? a_cols : a_rows;
  const int64_t n = transb ? b_cols : b_rows, kb = transb ? b_rows : b_cols;
  DH_CHECK(k == kb, "inner sizes differ: A gives k=%lld, B gives k=%lld", (long long)k, (long long)kb);
  if (m == 0 || n == 0) return DH_OK;
  DH_CHECK(d, "null output");
  DH_CHECK(k > 0 || accumulate, "empty inner dimension: D would be all zeros, clear it instead");
  if (k == 0) return DH_OK;                         // accumulating an empty sum
  DH_CHECK(a && b, "null operand");
  DH_CHECK(workspace || workspace_bytes == 0, "workspace_bytes given without a workspace");
  int dev = 0;
  DH_HIP(hipGetDevice(&dev));
  DH_CHECK(dev >= 0 && dev < 64, "device %d out of range", dev);
  Plan pl;
  hipblasLtHandle_t h;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_handle[dev]) DH_BLAS(hipblasLtCreate(&g_handle[dev]));
    h = g_handle[dev];
    const Key key{m, n, k, workspace_bytes, dev,
                  (transa ? 1 : 0) | (transb ? 2 : 0) | (accumulate ? 4 : 0) | (dtype << 3) | (out_dtype << 6)};
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
      Plan fresh;
      const int rc = make_plan(h, key, transa, transb, dtype, out_dtype, fresh);
      if (rc != DH_OK) return rc;
      it = g_plans.emplace(key, fresh).first;
    }
    pl = it->second;
  }
  DH_CHECK(pl.ws_needed <= workspace_bytes, "the chosen kernel wants %zu workspace bytes, %zu given", pl.ws_needed,
           workspace_bytes);
  const float one = 1.0f, zero = 0.0f;
  DH_BLAS(hipblasLtMatmul(h, pl.op, &one, a, pl.a, b, pl.b, accumulate ? &one : &zero, d, pl.d, d, pl.d, &pl.algo,
                          workspace, workspace_bytes, (hipStream_t)stream));
  return DH_OK;
}

extern "C" int dh_gemm(const void *a, const void *b, void *d, int64_t a_rows, int64_t a_cols, int64_t b_rows,
                       int64_t b_cols, int transa, int transb, int accumulate, int dtype, int out_dtype,
                       void *workspace, size_t workspace_bytes, void *stream) {
  DH_CHECK(!(transa && transb), "TT layout not allowed");
  return gemm_entry(a, b, d, a_rows, a_cols, b_rows, b_cols, transa, transb, accumulate, dtype, out_dtype, workspace,
                    workspace_bytes, stream);
}

// The layout dh_gemm refuses: D [n, m] = B^T @ A^T for A [m, k] and B [k, n], i.e. the weight-gradient product
// dW = dY^T X with X handed over transposed (A = X^T) and dY as it is.
extern "C" int dh_gemm_tt(const void *a, const void *b, void *d, int64_t a_rows, int64_t a_cols, int64_t b_rows,
                          int64_t b_cols, int accumulate, int dtype, int out_dtype, void *workspace,
                          size_t workspace_bytes, void *stream) {
  return gemm_entry(a, b, d, a_rows, a_cols, b_rows, b_cols, 1, 1, accumulate, dtype, out_dtype, workspace,
                    workspace_bytes, stream);
}

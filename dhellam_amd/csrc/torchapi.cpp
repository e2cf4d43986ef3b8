// pybind11 torch extension `dhellam._Clib`: the six names of the reference's native module
// (csrc/torchapi.cpp:2-9) with the argument order and return conventions of csrc/operators/ops.h:18-81,
// over the C ABI of libdhellam_hip.so (include/dhellam_hip.h).  at::Tensor stays on this side of the
// boundary: the library sees device pointers, sizes and a hipStream_t.
//
// Host code only (no kernels): built with the host compiler against torch's headers and linked with
// libdhellam_hip.so (dhellam_amd/build.py: build_torch_extension).
#include <torch/extension.h>
#include <c10/hip/HIPCachingAllocator.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "dhellam_hip.h"

namespace {

int dt(const at::Tensor &t) {
  switch (t.scalar_type()) {
    case at::kFloat: return DH_F32;
    case at::kBFloat16: return DH_BF16;
    case at::kHalf: return DH_F16;
    default: TORCH_CHECK(false, "dhellam._Clib: unsupported dtype ", t.scalar_type());
  }
}

void check(int rc) { TORCH_CHECK(rc == 0, "dhellam_hip error ", rc, ": ", dh_last_error()); }

void hip_check(hipError_t e) { TORCH_CHECK(e == hipSuccess, "HIP error: ", hipGetErrorString(e)); }

void need_gpu(std::initializer_list<const at::Tensor *> ts) {
  for (const at::Tensor *t : ts) TORCH_CHECK(t->is_cuda(), "dhellam._Clib: tensors must be on the GPU");
}

int64_t token_stride(const at::Tensor &t) {
  TORCH_CHECK(t.dim() == 3 && t.stride(2) == 1 && t.stride(1) == t.size(2),
              "attention tensors must be [tokens, heads, d] with contiguous (heads, d)");
  return t.stride(0);
}

// Elapsed milliseconds of `fn` on `stream` when profiling (events around it and a wait for the second one, as
// the reference does with cudaEvent, csrc/operators/gemm.cu:101-131); 0 and no synchronisation otherwise.
template <typename F> float timed(bool profiling, hipStream_t stream, F &&fn) {
  if (!profiling) {
    fn();
    return 0.f;
  }
  hipEvent_t a, b;
  hip_check(hipEventCreate(&a));
  hip_check(hipEventCreate(&b));
  hip_check(hipEventRecord(a, stream));
  fn();
  hip_check(hipEventRecord(b, stream));
  hip_check(hipEventSynchronize(b));
  float ms = 0.f;
  hip_check(hipEventElapsedTime(&ms, a, b));
  (void)hipEventDestroy(a);
  (void)hipEventDestroy(b);
  return ms;
}

// math_sm_count != 0: the call runs on a library-owned stream bound to |count| compute units (the first ones for
// a positive count, the last ones for a negative one; spread round-robin over the 8 XCDs), ordered after and
// before the caller's stream with events: what libsmctrl's next-launch mask does in the reference
// (csrc/operators/gemm.cu:66-70, smctrl.cpp:135-160).
hipStream_t masked_stream(int device, int count) {
  static std::mutex mu;
  static std::map<std::pair<int, int>, hipStream_t> cache;
  std::lock_guard<std::mutex> lock(mu);
  auto key = std::make_pair(device, count);
  auto it = cache.find(key);
  if (it != cache.end()) return it->second;
  hipDeviceProp_t prop;
  hip_check(hipGetDeviceProperties(&prop, device));
  const int n_cus = prop.multiProcessorCount, n = count < 0 ? -count : count;
  TORCH_CHECK(n > 0 && n <= n_cus, "math_sm_count=", count, " outside the ", n_cus, " compute units of this device");
  // bit i of the mask is compute unit i / 8 of XCD i % 8; take `n` units starting at `first`
  const int first = count > 0 ? 0 : n_cus - n;
  std::vector<uint32_t> words((n_cus + 31) / 32, 0u);
  for (int i = first; i < first + n; ++i) words[i / 32] |= 1u << (i % 32);
  void *st = nullptr;
  check(dh_stream_create_cu_mask(words.data(), (int)words.size(), &st));
  cache[key] = (hipStream_t)st;
  return (hipStream_t)st;
}

template <typename F> void confined(hipStream_t stream, int device, int math_sm_count, F &&launch) {
  if (math_sm_count == 0) {
    launch(stream);
    return;
  }
  hipStream_t m = masked_stream(device, math_sm_count);
  hipEvent_t e;
  hip_check(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  hip_check(hipEventRecord(e, stream));
  hip_check(hipStreamWaitEvent(m, e, 0));
  launch(m);
  hip_check(hipEventRecord(e, m));
  hip_check(hipStreamWaitEvent(stream, e, 0));
  (void)hipEventDestroy(e);     // the runtime keeps the event alive until the waits recorded on it are done
}

// A tensor allocated on torch's current stream and used on another raw stream: tell the caching allocator.
void record_on(const at::Tensor &t, hipStream_t stream) {
  if (stream == c10::hip::getCurrentHIPStream().stream()) return;
  c10::hip::HIPCachingAllocator::recordStream(t.storage().data_ptr(),
                                              c10::hip::getStreamFromExternal(stream, t.device().index()));
}

// Head dims the 16-bit kernels are compiled for; other sizes up to 256 run zero-padded to the next one (the reference
// pads to a multiple of 8 the same way, flash_atten.cu:303-312); fp32 takes any size as it is.
int64_t kernel_head_dim(const at::Tensor &t) {
  const int64_t d = t.size(-1);
  if (t.scalar_type() == at::kFloat) return d;
  for (int64_t s : {64, 96, 128, 192, 256})
    if (d <= s) return s;
  TORCH_CHECK(false, "attention supports head dims up to 256 (got ", d, ")");
}

at::Tensor pad_head_dim(const at::Tensor &t, int64_t d_to) {
  if (t.size(-1) == d_to) return t;
  return at::constant_pad_nd(t, {0, d_to - t.size(-1)}, 0);
}

at::Tensor ms_tensor(float ms) { return at::full({1}, ms, at::TensorOptions().dtype(at::kFloat)); }

}  // namespace

// csrc/operators/ops.h:18-32; flash_atten.cu:436-477 -> mha_varlen_fwd (:220-434).  Runs on torch's current
// stream.  Returns [out, q, k, v, out, softmax_lse, p, rng_state] (+ a CPU fp32 [1] tensor of milliseconds when
// profiling), the positions of flash_atten.cu:429-433; the supported head dims need no padding, so the "padded"
// slots hold the inputs themselves; p is empty and rng_state zero (no dropout).
std::vector<at::Tensor> pymha_varlen_fwd(const at::Tensor &q_in, const at::Tensor &k_in, const at::Tensor &v_in,
                                         const at::Tensor &cu_seqlens_q, const at::Tensor &cu_seqlens_k,
                                         int max_seqlen_q, int max_seqlen_k, float p_dropout, float softmax_scale,
                                         bool is_causal, bool return_softmax, int math_sm_count, bool profiling) {
  TORCH_CHECK(p_dropout == 0.f, "pymha_varlen_fwd: dropout is not implemented (p_dropout must be 0)");
  TORCH_CHECK(!return_softmax, "pymha_varlen_fwd: return_softmax is only supported with dropout in the reference");
  need_gpu({&q_in, &k_in, &v_in, &cu_seqlens_q, &cu_seqlens_k});
  TORCH_CHECK(cu_seqlens_q.scalar_type() == at::kInt && cu_seqlens_k.scalar_type() == at::kInt, "cu_seqlens must be int32");
  const int b = (int)cu_seqlens_q.numel() - 1;
  const int64_t d_og = q_in.size(-1), d_run = kernel_head_dim(q_in);
  const at::Tensor q = pad_head_dim(q_in, d_run), k = pad_head_dim(k_in, d_run), v = pad_head_dim(v_in, d_run);
  auto out_padded = at::empty(q.sizes(), q.options());
  auto lse = at::empty({b, q.size(1), max_seqlen_q}, q.options().dtype(at::kFloat));
  hipStream_t stream = c10::hip::getCurrentHIPStream().stream();
  const float ms = timed(profiling, stream, [&] {
    confined(stream, q.device().index(), math_sm_count, [&](hipStream_t st) {
      check(dh_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out_padded.data_ptr(), lse.data_ptr<float>(),
                        cu_seqlens_q.data_ptr<int>(), cu_seqlens_k.data_ptr<int>(), b, max_seqlen_q, max_seqlen_k,
                        (int)q.size(1), (int)k.size(1), (int)q.size(2), token_stride(q), token_stride(k),
                        token_stride(v), token_stride(out_padded), softmax_scale, is_causal ? 1 : 0, dt(q), st));
    });
  });
  const at::Tensor out = d_run == d_og ? out_padded : out_padded.narrow(-1, 0, d_og);
  std::vector<at::Tensor> res = {out, q, k, v, out_padded, lse, at::empty({0}, q.options()),
                                 at::zeros({2}, q.options().dtype(at::kLong))};
  if (profiling) res.push_back(ms_tensor(ms));
  return res;
}

// csrc/operators/ops.h:34-52; flash_atten.cu:760-813 -> mha_varlen_bwd (:479-757).  Unlike the forward it
// launches on the raw stream its caller hands over (flash_atten.cu:784; 0 = torch's current stream).  Returns
// [dq, dk, dv, softmax_d] (+ the milliseconds tensor when profiling).  The result does not depend on
// `deterministic`: no floating-point atomics are used either way.
std::vector<at::Tensor> pymha_varlen_bwd(const at::Tensor &dout_in, const at::Tensor &q_in, const at::Tensor &k_in,
                                         const at::Tensor &v_in, const at::Tensor &out_in, const at::Tensor &softmax_lse,
                                         const at::Tensor &cu_seqlens_q, const at::Tensor &cu_seqlens_k,
                                         int max_seqlen_q, int max_seqlen_k, float p_dropout, float softmax_scale,
                                         bool is_causal, c10::optional<at::Tensor> rng_state, bool deterministic,
                                         int math_sm_count, bool profiling, uint64_t stream_ptr) {
  (void)rng_state;
  (void)deterministic;
  TORCH_CHECK(p_dropout == 0.f, "pymha_varlen_bwd: dropout is not implemented (p_dropout must be 0)");
  need_gpu({&dout_in, &q_in, &k_in, &v_in, &out_in, &softmax_lse, &cu_seqlens_q, &cu_seqlens_k});
  TORCH_CHECK(softmax_lse.scalar_type() == at::kFloat && softmax_lse.is_contiguous(), "softmax_lse must be contiguous fp32");
  const int64_t d_og = q_in.size(-1), d_run = kernel_head_dim(q_in);
  const at::Tensor dout = pad_head_dim(dout_in, d_run), q = pad_head_dim(q_in, d_run), k = pad_head_dim(k_in, d_run),
                   v = pad_head_dim(v_in, d_run), out = pad_head_dim(out_in, d_run);
  const int b = (int)cu_seqlens_q.numel() - 1, hq = (int)q.size(1), hk = (int)k.size(1), d = (int)q.size(2);
  auto dq = at::empty(q.sizes(), q.options()), dk = at::empty(k.sizes(), k.options()), dv = at::empty(v.sizes(), v.options());
  auto softmax_d = at::zeros({b, hq, max_seqlen_q}, q.options().dtype(at::kFloat));
  // scratch: the library says how much, and is told how much it got
  const size_t ws_bytes = dh_attn_bwd_workspace_bytes(q.size(0), k.size(0), b, max_seqlen_q, hq, hk, d, dt(q));
  auto ws = at::empty({(int64_t)ws_bytes}, q.options().dtype(at::kByte));
  hipStream_t stream = stream_ptr ? (hipStream_t)stream_ptr : c10::hip::getCurrentHIPStream().stream();
  if (stream_ptr) {
    // outputs and scratch come from torch's current stream: the raw stream must not run ahead of their allocation
    // (a block just freed by earlier work on the current stream), and the allocator must know who uses them
    hipStream_t cur = c10::hip::getCurrentHIPStream().stream();
    if (cur != stream) {
      hipEvent_t e;
      hip_check(hipEventCreateWithFlags(&e, hipEventDisableTiming));
      hip_check(hipEventRecord(e, cur));
      hip_check(hipStreamWaitEvent(stream, e, 0));
      (void)hipEventDestroy(e);
    }
  }
  const float ms = timed(profiling, stream, [&] {
    confined(stream, q.device().index(), math_sm_count, [&](hipStream_t st) {
      check(dh_attn_bwd(dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                        softmax_lse.data_ptr<float>(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                        softmax_d.data_ptr<float>(), ws.data_ptr(), ws_bytes, cu_seqlens_q.data_ptr<int>(),
                        cu_seqlens_k.data_ptr<int>(), b, max_seqlen_q, max_seqlen_k, q.size(0), k.size(0), hq, hk, d,
                        token_stride(q), token_stride(k), token_stride(v), token_stride(out), token_stride(dout),
                        token_stride(dq), token_stride(dk), token_stride(dv), softmax_scale, is_causal ? 1 : 0,
                        dt(q), st));
    });
  });
  for (const at::Tensor *t : std::initializer_list<const at::Tensor *>{&ws, &dq, &dk, &dv, &softmax_d, &dout, &q, &k, &v, &out})
    record_on(*t, stream);
  if (d_run != d_og) {       // the gradients of the columns that were given
    c10::hip::HIPStreamGuard guard(c10::hip::getStreamFromExternal(stream, q.device().index()));
    dq = dq.narrow(-1, 0, d_og).contiguous();
    dk = dk.narrow(-1, 0, d_og).contiguous();
    dv = dv.narrow(-1, 0, d_og).contiguous();
  }
  std::vector<at::Tensor> res = {dq, dk, dv, softmax_d};
  if (profiling) res.push_back(ms_tensor(ms));
  return res;
}

// csrc/operators/ops.h:54-65; gemm.cu:133-170 (pygemm -> cublas_gemm, :3-131).  Column-major library
// convention over row-major tensors: D = op(B) @ op(A), i.e. transa ("TN") B @ A^T, neither ("NN") B @ A,
// transb ("NT") B^T @ A; both is refused as in the reference.
float pygemm(const at::Tensor &inputA, const at::Tensor &inputB, at::Tensor &outputD, at::Tensor &input_workspace,
             size_t workspaceSize, bool transa, bool transb, bool grad_accumulate, int math_sm_count,
             bool profiling) {
  TORCH_CHECK(!(transa && transb), "pygemm: TT layout not allowed");
  need_gpu({&inputA, &inputB, &outputD, &input_workspace});
  TORCH_CHECK(inputA.dim() == 2 && inputB.dim() == 2 && outputD.dim() == 2 && inputA.is_contiguous() &&
                  inputB.is_contiguous() && outputD.is_contiguous(),
              "pygemm: operands must be contiguous 2-D tensors");
  TORCH_CHECK((size_t)input_workspace.nbytes() >= workspaceSize, "pygemm: workspace tensor smaller than workspaceSize");
  hipStream_t stream = c10::hip::getCurrentHIPStream().stream();
  return timed(profiling, stream, [&] {
    confined(stream, inputA.device().index(), math_sm_count, [&](hipStream_t st) {
      check(dh_gemm(inputA.data_ptr(), inputB.data_ptr(), outputD.data_ptr(), inputA.size(0), inputA.size(1),
                    inputB.size(0), inputB.size(1), transa ? 1 : 0, transb ? 1 : 0, grad_accumulate ? 1 : 0,
                    dt(inputA), dt(outputD), input_workspace.data_ptr(), workspaceSize, st));
    });
  });
}

// csrc/operators/ops.h:71-76; gelu.cu:17-43 (tanh-approximation GELU into `output`).
float pygelu(const at::Tensor &input, at::Tensor &output, bool profiling) {
  need_gpu({&input, &output});
  TORCH_CHECK(input.is_contiguous() && output.is_contiguous() && input.numel() == output.numel(), "pygelu: shapes");
  hipStream_t stream = c10::hip::getCurrentHIPStream().stream();
  return timed(profiling, stream, [&] {
    check(dh_gelu(input.data_ptr(), output.data_ptr(), input.numel(), dt(input), stream));
  });
}

// csrc/operators/ops.h:78-81; bda.cu:18-62: output = mask * (input + bias) + residual with the mask all ones
// (the reference draws it with torch::dropout; only prob = 0 is implemented).
float pybda(const at::Tensor &input, const at::Tensor &bias, const at::Tensor &residual, at::Tensor &output,
            float prob, bool profiling) {
  TORCH_CHECK(prob == 0.f, "pybda: only prob = 0 is implemented");
  need_gpu({&input, &bias, &residual, &output});
  hipStream_t stream = c10::hip::getCurrentHIPStream().stream();
  return timed(profiling, stream, [&] {
    check(dh_bias_mask_add(input.data_ptr(), bias.data_ptr(), residual.data_ptr(), nullptr, output.data_ptr(),
                           input.numel(), dt(input), stream));
  });
}

// csrc/operators/ops.h:67-69.
at::Tensor add_tensors(const at::Tensor &a, const at::Tensor &b) { return a + b; }

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  namespace py = pybind11;
  m.doc() = "dhellam._Clib over libdhellam_hip.so (MI355X): the six names of the reference's extension";
  m.def("add_tensors", &add_tensors, "add", py::arg("a"), py::arg("b"));
  m.def("pygemm", &pygemm, "gemm", py::arg("inputA"), py::arg("inputB"), py::arg("outputD"),
        py::arg("input_workspace"), py::arg("workspaceSize"), py::arg("transa"), py::arg("transb"),
        py::arg("grad_accumulate"), py::arg("math_sm_count"), py::arg("profiling"));
  m.def("pygelu", &pygelu, "gelu", py::arg("input"), py::arg("output"), py::arg("profiling"));
  m.def("pybda", &pybda, "bda", py::arg("input"), py::arg("bias"), py::arg("residual"), py::arg("output"),
        py::arg("prob"), py::arg("profiling"));
  m.def("pymha_varlen_fwd", &pymha_varlen_fwd, "mha_varlen_fwd", py::arg("q"), py::arg("k"), py::arg("v"),
        py::arg("cu_seqlens_q"), py::arg("cu_seqlens_k"), py::arg("max_seqlen_q"), py::arg("max_seqlen_k"),
        py::arg("p_dropout"), py::arg("softmax_scale"), py::arg("is_causal"), py::arg("return_softmax"),
        py::arg("math_sm_count"), py::arg("profiling"));
  m.def("pymha_varlen_bwd", &pymha_varlen_bwd, "mha_varlen_bwd", py::arg("dout"), py::arg("q"), py::arg("k"),
        py::arg("v"), py::arg("out"), py::arg("softmax_lse"), py::arg("cu_seqlens_q"), py::arg("cu_seqlens_k"),
        py::arg("max_seqlen_q"), py::arg("max_seqlen_k"), py::arg("p_dropout"), py::arg("softmax_scale"),
        py::arg("is_causal"), py::arg("rng_state"), py::arg("deterministic"), py::arg("math_sm_count"),
        py::arg("profiling"), py::arg("stream_ptr"));
}

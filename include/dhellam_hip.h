/*
 * dhellam_hip.h -- C ABI of the MI355X (gfx950) operator library behind the
 * DHeLlam per-rank operator hot path.
 *
 * Every entry point takes raw DEVICE pointers, plain sizes and a HIP stream
 * handle (hipStream_t passed as void*; NULL = the null stream).  All kernels
 * are enqueued asynchronously on that stream; nothing here synchronises and,
 * unless an entry says so, nothing here allocates.  Return value: 0 on
 * success, a negative dh_status otherwise; dh_last_error() then holds a
 * "file:line in function: message" string for the calling thread (the
 * reference's DHELLAM_CHECK style, csrc/operators/logging.h:53-86, without the
 * C++ exception).
 *
 * The reference binds this path through a pybind11 torch extension
 * (csrc/torchapi.cpp:2-9, csrc/operators/ops.h:18-81); each declaration below
 * cites the reference interface it stands behind.  The Python mirror of that
 * extension (dhellam_amd/_Clib.py) is a thin ctypes shim over these symbols.
 */
#ifndef DHELLAM_HIP_H
#define DHELLAM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { DH_F32 = 0, DH_BF16 = 1, DH_F16 = 2 } dh_dtype;

typedef enum {
  DH_OK = 0,
  DH_ERR_INVALID = -1,   /* bad argument / unsupported shape */
  DH_ERR_HIP = -2,       /* a HIP runtime call failed */
  DH_ERR_UNSUPPORTED = -3
} dh_status;

/* Library version (major*100 + minor).  2.0: dh_attn_bwd, dh_attn_bwd_acc,
 * dh_norm_bwd and dh_moe_sort take the size of the caller's workspace and
 * check it (1.x trusted the caller); dh_grouped_gemm_nt / _nn take an optional
 * workspace. */
int dh_version(void);
/* Message of the last failing call on this thread ("" if none). */
const char *dh_last_error(void);

/* ------------------------------------------------------------------------
 * Normalisation.  Stands behind dhellam/operators/layernorm.py:6-45
 * (pylayernorm_fwd -> tex.layernorm_fwd) and :47-91 (pylayernorm_bwd ->
 * tex.layernorm_bwd).  beta == NULL selects RMSNorm (y = x * rsigma * gamma,
 * mu unused); beta != NULL selects LayerNorm (y = (x-mu)*rsigma*gamma+beta).
 * x, y, gamma, beta share `dtype`; mu/rsigma are fp32 [rows].
 * zero_centered_gamma: gamma is stored as (gamma - 1).
 * ---------------------------------------------------------------------- */
int dh_norm_fwd(const void *x, const void *gamma, const void *beta, void *y,
                float *mu, float *rsigma, int64_t rows, int64_t cols,
                float eps, int zero_centered_gamma, int dtype, void *stream);

/* The residual add of the reference's bda operator (dhellam/operators/bda.py:3-7 with the dropout mask all ones,
 * dhellam/core/dstb.py:273-277) and the norm that follows it (dstb.py:73-78) in one pass:
 * sum_out = x + residual (rounded to `dtype`, exactly what dh_residual_add stores) and y = norm(sum_out).
 * The two ops are adjacent in the layer (bda_attn, ln_mlp); fused, the sum is not read back from memory and
 * one launch goes away.  sum_out may alias x or residual. */
int dh_add_norm_fwd(const void *x, const void *residual, void *sum_out,
                    const void *gamma, const void *beta, void *y, float *mu,
                    float *rsigma, int64_t rows, int64_t cols, float eps,
                    int zero_centered_gamma, int dtype, void *stream);

/* Bytes of fp32 scratch dh_norm_bwd needs for its dgamma/dbeta partial sums. */
size_t dh_norm_bwd_workspace_bytes(int64_t rows, int64_t cols);

/* dx = d(loss)/dx (+ add_to_dx if non-NULL: the residual-branch gradient the
 * reference adds in a separate launch, dhellam/core/dstb.py:387-405).
 * dgamma/dbeta [cols] in `dtype`; mu == NULL selects RMSNorm (dbeta may be
 * NULL).  accumulate_wgrad != 0: dgamma/dbeta are added to instead of
 * overwritten.  workspace: workspace_bytes bytes, at least
 * dh_norm_bwd_workspace_bytes(rows, cols) or the call is refused with
 * DH_ERR_INVALID before anything is launched. */
int dh_norm_bwd(const void *dy, const void *x, const float *mu,
                const float *rsigma, const void *gamma, const void *add_to_dx,
                void *dx, void *dgamma, void *dbeta, void *workspace,
                size_t workspace_bytes, int64_t rows, int64_t cols,
                int zero_centered_gamma, int accumulate_wgrad, int dtype,
                void *stream);

/* ------------------------------------------------------------------------
 * SwiGLU.  dhellam/operators/swiglu.py:13-16 (fwd) and :21-26 (bwd).
 * y [rows, 2*f]: gate = first f columns, up = last f.  out [rows, f].
 * bwd: dy [rows, 2*f] = cat(g*sig(y1)*(1+y1*(1-sig(y1)))*y2, g*silu(y1)).
 * ---------------------------------------------------------------------- */
int dh_swiglu_fwd(const void *y, void *out, int64_t rows, int64_t f, int dtype,
                  void *stream);
int dh_swiglu_bwd(const void *g, const void *y, void *dy, int64_t rows,
                  int64_t f, int dtype, void *stream);

/* dh_swiglu_fwd that also writes its result transposed: out_t [f, rows]
 * (row-major) next to out [rows, f], for the weight-gradient product of the
 * projection behind the activation (dhellam/core/dstb.py:543-598), which runs
 * with the activation handed over transposed (dh_gemm_tt).  16-bit types; rows
 * and f multiples of 8; out is bit for bit that of dh_swiglu_fwd.  No
 * counterpart in the reference. */
int dh_swiglu_fwd_t(const void *y, void *out, void *out_t, int64_t rows,
                    int64_t f, int dtype, void *stream);

/* dh_swiglu_bwd that also writes the gradient transposed: dy_t [2f, rows]
 * (row-major) next to dy [rows, 2f], for the weight-gradient product of the
 * projection in front of the activation (csrc/operators/gemm.cu:3-170 with
 * transb; dhellam/core/dstb.py:543-598).  16-bit types; rows and f multiples
 * of 8.  No counterpart in the reference. */
int dh_swiglu_bwd_t(const void *g, const void *y, void *dy, void *dy_t,
                    int64_t rows, int64_t f, int dtype, void *stream);

/* ------------------------------------------------------------------------
 * Residual add (bias-dropout-add with dropout disabled).
 * dhellam/operators/bda.py:3-12.  out = x + residual (out may alias x: the
 * reference op is in-place on its input).  n = element count.
 * ---------------------------------------------------------------------- */
int dh_residual_add(const void *x, const void *residual, void *out, int64_t n,
                    int dtype, void *stream);

/* Legacy elementwise kernels of the binding surface, fp16/bf16/fp32.
 * csrc/operators/gelu.cu:10-15 (tanh GELU) and csrc/operators/bda.cu:10-16
 * (out = mask*(x+bias)+residual; mask == NULL means all-ones). */
int dh_gelu(const void *x, void *out, int64_t n, int dtype, void *stream);
int dh_bias_mask_add(const void *x, const void *bias, const void *residual,
                     const void *mask, void *out, int64_t n, int dtype,
                     void *stream);

/* ------------------------------------------------------------------------
 * Rotary position embedding (rotate-half, non-interleaved).  The reference has
 * no RoPE; its slot is between the q/k/v split and the attention call
 * (dhellam/core/dstb.py:122-126) and, in backward, before the dq/dk/dv concat
 * (:376-382).  q [tokens, hq, d], k [tokens, hk, d] (k may be NULL), token
 * stride given in elements so q/k may be views into a packed qkv row.
 * inv_freq: fp32 [d/2] on device; angle = (float)pos * inv_freq[j].
 * positions: int32 [tokens] or NULL (then pos = t % seq_len, or t if
 * seq_len <= 0).  backward != 0 applies the inverse rotation (sin -> -sin).
 * Output may alias input.
 * ---------------------------------------------------------------------- */
int dh_rope(const void *q, const void *k, void *q_out, void *k_out,
            const float *inv_freq, const int32_t *positions, int64_t tokens,
            int hq, int hk, int d, int64_t q_stride, int64_t k_stride,
            int64_t qo_stride, int64_t ko_stride, int64_t seq_len,
            int backward, int dtype, void *stream);

/* ------------------------------------------------------------------------
 * Variable-length flash attention.  csrc/operators/ops.h:18-32 /
 * csrc/operators/flash_atten.cu:220-434 (forward) and ops.h:34-52 /
 * flash_atten.cu:479-757 (backward).
 * q [total_q, hq, d], k/v [total_k, hk, d], out like q; token strides are in
 * elements (head stride is d, last dim contiguous).  cu_seqlens_* int32 [b+1]
 * on device.  lse fp32 [b, hq, max_seqlen_q] = natural-log logsumexp of the
 * scaled scores (-inf rows never occur for causal sq == sk).  causal requires
 * per-sequence sq == sk.  hq % hk == 0 (GQA).  d in {64, 96, 128, 192, 256}
 * for bf16/fp16 (the reference takes any d <= 256 and pads it to a multiple
 * of 8 above this boundary, flash_atten.cu:284,303-312: a binding pads other
 * sizes with zero columns to the next of these, as dhellam._Clib does), any
 * d <= 256 with d % 4 == 0 for fp32.
 * ---------------------------------------------------------------------- */
int dh_attn_fwd(const void *q, const void *k, const void *v, void *out,
                float *lse, const int32_t *cu_seqlens_q,
                const int32_t *cu_seqlens_k, int batch, int max_seqlen_q,
                int max_seqlen_k, int hq, int hk, int d, int64_t q_stride,
                int64_t k_stride, int64_t v_stride, int64_t o_stride,
                float softmax_scale, int causal, int dtype, void *stream);

/* Bytes of scratch dh_attn_bwd works in.  dh_attn_bwd_min_workspace_bytes: what
 * every call of these sizes needs (delta = rowsum(dO*O), the lse / delta planes
 * of the head-dim-128 kernels, fp32 dK/dV partials when a GQA group is split
 * over workgroups); a smaller workspace is refused.  dh_attn_bwd_workspace_bytes:
 * that plus room for the dS blocks of calls that would keep them (below); with
 * it the backward picks its faster form. */
size_t dh_attn_bwd_min_workspace_bytes(int64_t total_q, int64_t total_k,
                                       int batch, int max_seqlen_q, int hq,
                                       int hk, int d, int dtype);
size_t dh_attn_bwd_workspace_bytes(int64_t total_q, int64_t total_k, int batch,
                                   int max_seqlen_q, int hq, int hk, int d,
                                   int dtype);

/* Head dim 128 in 16 bits, calls too small to fill the chip with 128-row
 * query tiles (fewer than 256 of them, halved for causal): the backward keeps
 * dS = P * (dP - delta) from its dK/dV pass and forms dQ from it in one
 * product when 2 bytes per (head, query, key) (a) stay under this process-wide
 * limit (default 1280 MiB; 0: never keep) and (b) fit into the workspace the
 * call was given behind its minimum; otherwise its dQ pass recomputes S and dP
 * and needs no such space.  The limit only steers the choice: a call never
 * writes past workspace + workspace_bytes, whatever the limit is or was when
 * the workspace was sized.  No counterpart in the reference (flash-attention
 * always recomputes). */
void dh_attn_bwd_set_ds_limit(size_t bytes);
/* on != 0: calls large enough to fill the chip with the recomputing dQ kernel
 * keep dS as well (same limit, same workspace check).  Process-wide. */
void dh_attn_bwd_set_ds_when_full(int on);

/* dq like q, dk/dv like k/v (GQA groups are reduced inside the kernel; the
 * reference sums an expanded buffer afterwards, flash_atten.cu:646-652).
 * delta_out (fp32 [b, hq, max_seqlen_q], may be NULL) receives rowsum(dO*O),
 * the reference's softmax_d, for the rows of each sequence (entries past a
 * sequence's length are left as they were).  workspace: workspace_bytes bytes,
 * 16-byte aligned; fewer than dh_attn_bwd_min_workspace_bytes() is refused
 * with DH_ERR_INVALID before anything is launched. */
int dh_attn_bwd(const void *dout, const void *q, const void *k, const void *v,
                const void *out, const float *lse, void *dq, void *dk,
                void *dv, float *delta_out, void *workspace,
                size_t workspace_bytes,
                const int32_t *cu_seqlens_q, const int32_t *cu_seqlens_k,
                int batch, int max_seqlen_q, int max_seqlen_k,
                int64_t total_q, int64_t total_k, int hq, int hk, int d,
                int64_t q_stride, int64_t k_stride, int64_t v_stride,
                int64_t o_stride, int64_t do_stride, int64_t dq_stride,
                int64_t dk_stride, int64_t dv_stride, float softmax_scale,
                int causal, int dtype, void *stream);

/* dh_attn_bwd with one more argument: accumulate_dq != 0 adds this call's dq
 * to the values already in `dq` (read, added in fp32, rounded once) instead of
 * overwriting them: a ring step's `dq.add_(dq_)` of
 * dhellam/operators/ring_attn.py:391-408 without the temporary and the extra
 * pass.  dk/dv are written as in dh_attn_bwd. */
int dh_attn_bwd_acc(const void *dout, const void *q, const void *k,
                    const void *v, const void *out, const float *lse, void *dq,
                    void *dk, void *dv, float *delta_out, void *workspace,
                    size_t workspace_bytes,
                    const int32_t *cu_seqlens_q, const int32_t *cu_seqlens_k,
                    int batch, int max_seqlen_q, int max_seqlen_k,
                    int64_t total_q, int64_t total_k, int hq, int hk, int d,
                    int64_t q_stride, int64_t k_stride, int64_t v_stride,
                    int64_t o_stride, int64_t do_stride, int64_t dq_stride,
                    int64_t dk_stride, int64_t dv_stride, float softmax_scale,
                    int causal, int accumulate_dq, int dtype, void *stream);

/* ------------------------------------------------------------------------
 * Ring-attention merge of per-step partial results.
 * dhellam/operators/ring_attn.py:26-40 (lse and out correction) applied as in
 * :146-195, in one pass and in fp32.  Step s contributes rows
 * [row_begin[s], row_begin[s]+rows[s]) of every sequence (the reference's
 * "second half of q" steps have row_begin = sq/2).  outs[s]: [b*rows[s], hq,
 * d] contiguous; lses[s]: fp32 [b, hq, rows[s]].  out [b*sq, hq, d];
 * lse fp32 [b, hq, sq].  n_steps <= 8.  Host arrays of device pointers.
 * ---------------------------------------------------------------------- */
int dh_attn_merge(const void *const *outs, const float *const *lses,
                  const int32_t *row_begin, const int32_t *rows, int n_steps,
                  void *out, float *lse, int batch, int sq, int hq, int d,
                  int dtype, void *stream);

/* ------------------------------------------------------------------------
 * MoE routing and token permutation.  No counterpart in the reference (it has
 * no MoE); semantics are Mixtral/Megatron-core dropless top-k routing.
 * ---------------------------------------------------------------------- */
/* logits fp32 [tokens, experts] -> topk_idx int32 [tokens, k] (descending
 * logit, ties to the lower expert id), gates fp32 [tokens, k] = softmax over
 * the k selected logits.  experts <= 64, k <= 8. */
int dh_moe_route_topk(const float *logits, int32_t *topk_idx, float *gates,
                      int64_t tokens, int experts, int k, void *stream);

size_t dh_moe_sort_workspace_bytes(int64_t n_assign, int experts);
/* Stable counting sort of the flat assignment list topk_idx [n_assign]
 * (assignment a = token*k + j) by expert id.  tokens_per_expert int32
 * [experts]; expert_offsets int32 [experts+1] (exclusive scan of the counts);
 * sorted_idx int32 [n_assign] (assignment ids in sorted order); dest_row int32
 * [n_assign] (position of each assignment in the sorted order).  workspace:
 * workspace_bytes bytes, at least dh_moe_sort_workspace_bytes(n_assign,
 * experts) or the call is refused with DH_ERR_INVALID. */
int dh_moe_sort(const int32_t *topk_idx, int32_t *tokens_per_expert,
                int32_t *expert_offsets, int32_t *sorted_idx, int32_t *dest_row,
                void *workspace, size_t workspace_bytes, int64_t n_assign,
                int experts, void *stream);

/* dh_moe_sort for callers that cannot allocate device memory or pass a workspace (code under HIP graph capture,
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same results as
 * dh_moe_sort; the per-block histogram table lives in a device array inside the library (256 KiB per GPU, held
 * until the process ends), so n_assign is limited to dh_moe_sort_static_max_assign() (2^20) and a larger list
 * is refused with DH_ERR_INVALID.  Calls no hipMalloc / hipFree.  Every call on a GPU uses that GPU's one
 * table: calls that overlap on one GPU (two streams) race; calls in stream order do not. */
int64_t dh_moe_sort_static_max_assign(void);
int dh_moe_sort_static(const int32_t *topk_idx, int32_t *tokens_per_expert,
                       int32_t *expert_offsets, int32_t *sorted_idx,
                       int32_t *dest_row, int64_t n_assign, int experts,
                       void *stream);

/* The rows of local experts [e_lo, e_hi) are the sorted positions
 * [first, first + n_rows) with first = expert_offsets[e_lo] and n_rows =
 * expert_offsets[e_hi] - first, both read ON DEVICE (no host sync); launches
 * cover max_rows / tokens.  `permuted` holds max_rows rows: rows past that are
 * never written, whatever the offsets say, and rows [n_rows, max_rows) are
 * zeroed (so `permuted` may be uninitialised on entry).
 *
 * gather: permuted[r] = scale * x[sorted_idx[first + r] / k] for r < n_rows,
 * scale = row_scale[sorted_idx[first + r]] if row_scale != NULL else 1. */
int dh_moe_gather_rows(const void *x, const int32_t *sorted_idx,
                       const float *row_scale, void *permuted,
                       const int32_t *expert_offsets, int e_lo, int e_hi,
                       int64_t max_rows, int k, int64_t hidden, int dtype,
                       void *stream);

/* scatter: out[t] = sum_j w(t,j) * y[dest_row[t*k+j] - first] over the j whose
 * sorted position is local; w = gates[t*k+j], or 1 if gates == NULL.  Tokens
 * with no local assignment get zeros.  j order is fixed (deterministic). */
int dh_moe_scatter_rows(const void *y, const int32_t *dest_row,
                        const float *gates, void *out,
                        const int32_t *expert_offsets, int e_lo, int e_hi,
                        int64_t tokens, int k, int64_t hidden, int dtype,
                        void *stream);

/* dgates[t*k+j] = <dout[t], y[dest_row[t*k+j]-first]> (0 if not local). */
int dh_moe_gate_grad(const void *dout, const void *y, const int32_t *dest_row,
                     float *dgates, const int32_t *expert_offsets, int e_lo,
                     int e_hi, int64_t tokens, int k, int64_t hidden, int dtype,
                     void *stream);

/* ------------------------------------------------------------------------
 * Grouped GEMM on MFMA (bf16/fp16 in, fp32 accumulate).  No counterpart in
 * the reference.  Group g owns rows [offs[g]-offs[0], offs[g+1]-offs[0]) of
 * the stacked row dimension (offs: device int32 [groups+1], read on device,
 * so a slice of expert_offsets can be passed as is).
 *   NT: c[rows_g, n] = a[rows_g, k] * b[g][n, k]^T          (forward)
 *   NN: c[rows_g, n] = a[rows_g, k] * b[g][k, n]            (dgrad)
 *   TN: c[g][m, n] (+)= a[rows_g, m]^T * b[rows_g, n]       (wgrad)
 * max_rows is the number of rows the stacked operands hold: it bounds the launch grid, group ranges read
 * from offs are cut off there (no row past it is read or written), and NT / NN zero the rows of c from the
 * last group's end up to max_rows, so c may be uninitialised on entry.
 * workspace (NT, NN; may be NULL): device memory of at least dh_grouped_gemm_workspace_bytes() bytes.  With it,
 * a product that fills the chip may have its last round of tiles split along k: the tiles run in rounds of one
 * per compute unit, and when the last round holds at most half as many tiles as there are compute units a second
 * kernel computes them in as many k pieces as fit, whose fp32 sums go through the workspace and are added in k order
 * by a third kernel (deterministic).  288 tiles on 256 compute units then cost 1 1/8 tile times instead of 2; when
 * nothing is split the two extra launches find nothing to do.  Without a workspace a
 * tile is one workgroup and the last round is as full as it happens to be.  The contents of the workspace do not
 * matter on entry; calls that overlap on one device need workspaces of their own.
 * ---------------------------------------------------------------------- */
size_t dh_grouped_gemm_workspace_bytes(void);
int dh_grouped_gemm_nt(const void *a, const void *b, void *c,
                       const int32_t *offs, int groups, int64_t max_rows,
                       int64_t n, int64_t k, int dtype, void *workspace,
                       size_t workspace_bytes, void *stream);
int dh_grouped_gemm_nn(const void *a, const void *b, void *c,
                       const int32_t *offs, int groups, int64_t max_rows,
                       int64_t n, int64_t k, int dtype, void *workspace,
                       size_t workspace_bytes, void *stream);
int dh_grouped_gemm_tn(const void *a, const void *b, void *c,
                       const int32_t *offs, int groups, int64_t max_rows,
                       int64_t m, int64_t n, int accumulate, int dtype,
                       void *stream);

/* Plain device-to-device copy kernel: a known-size streaming kernel used to
 * calibrate the profiler's HBM byte counters, and the local stand-in for the
 * sequence-parallel all-gather of the reference's communication operator
 * (dhellam/operators/comm.py, all_gather_into_tensor call sites in
 * dhellam/core/dstb.py) when one GPU holds the whole sequence. */
int dh_copy_bytes(const void *src, void *dst, int64_t nbytes, void *stream);

/* Keeps `stream` busy with a one-wavefront kernel for about `nanoseconds` (at most 1 s) without using the
 * memory system.  No counterpart in the reference: on one GPU it stands in for the DURATION of a collective
 * (dhellam/common/comm.py) in scheduler experiments, so that the double-strand runtime has something to hide. */
int dh_delay(int64_t nanoseconds, void *stream);

/* The same stretch of stream time spent in a host function of the stream
 * (hipLaunchHostFunc) instead of a kernel: stands for a transfer that needs no
 * compute unit (copy engine, network adapter), so it starts while kernels of
 * another stream fill the device.  No counterpart in the reference. */
int dh_host_delay(int64_t nanoseconds, void *stream);

/* ------------------------------------------------------------------------
 * Resident communication proxy: collectives that a stream posts and waits for
 * without a kernel launch per collective.  It stands where the reference has
 * its third stream and communication handles (dhellam/core/dstb.py:1142-1188:
 * the collective is posted on stream 3, the compute op waits for its handle);
 * the reference's collectives themselves (dhellam/operators/comm.py) are NCCL
 * kernels.  One kernel, launched at the start of a step, keeps one wavefront
 * per slot (a slot = a strand's communication channel) resident; a request is
 * posted with a stream write and waited for with a stream wait, both carried
 * out by the command processor, so a request is seen within microseconds even
 * while a kernel of another stream owns every compute unit (a collective
 * launched as a kernel of its own then waits until that kernel has placed its
 * last workgroup).  On one GPU a request is carried out by waiting
 * `duration_ns`.  All waits of the kernel are bounded (see launch).
 *
 * create: allocates the proxy (host object + three 8-byte pieces of signal
 *   memory per slot and a log, kept until the process ends); slots <= 8.
 * launch: starts the kernel on `stream` (a stream of its own, not a strand's).
 *   A slot that sees neither a request nor its stop for `limit_ns` gives up and
 *   releases every stream wait behind it.  One launch at a time.
 * post / wait: on the strand's stream; a wait refers to the slot's last post.
 * stop: streams[slot] = the stream whose order ends the slot's requests of
 *   this launch (the strand's stream); the kernel ends once every slot has
 *   seen its stop with nothing pending.
 * log: after the launch's streams have been synchronised, the (start, end)
 *   times in ns (a 100 MHz device clock, arbitrary origin) of up to
 *   max_entries collectives the slot carried out; clears the log.
 * ---------------------------------------------------------------------- */
int dh_comm_proxy_create(int slots, void **proxy_out);
int dh_comm_proxy_launch(void *proxy, int64_t duration_ns, int64_t limit_ns,
                         void *stream);
int dh_comm_proxy_post(void *proxy, int slot, void *stream);
int dh_comm_proxy_wait(void *proxy, int slot, void *stream);
int dh_comm_proxy_stop(void *proxy, const void *const *streams);
int dh_comm_proxy_log(void *proxy, int slot, int64_t max_entries,
                      int64_t *start_ns, int64_t *end_ns, int64_t *n_out);

/* Dense GEMM through hipBLASLt: cublas_gemm / pygemm, csrc/operators/gemm.cu:3-170 (csrc/operators/ops.h:54-65).
 * The reference's convention is kept: A [a_rows, a_cols], B [b_rows, b_cols] and D are contiguous row-major
 * arrays given to a column-major library, so with m = transa ? a_rows : a_cols, k = transa ? a_cols : a_rows,
 * n = transb ? b_cols : b_rows the result is the row-major D [n, m] =
 *   transa=1, transb=0: B @ A^T (forward: activations x weight^T)     transa=0, transb=0: B @ A (data gradient)
 *   transa=0, transb=1: B^T @ A (weight gradient)                      transa=1, transb=1: refused, as there.
 * `accumulate` (the reference's grad_accumulate) adds to D instead of overwriting it.  Operands are bf16 / fp16
 * / fp32 (`dtype`), D is of the same type or fp32 (`out_dtype`); products are accumulated in fp32.
 * `workspace` (device, 256-byte aligned) and its size are what the library may use, as in the reference;
 * the kernel is chosen once per (shape, layout, types, workspace size, device) by the library's heuristic and
 * cached.  `math_sm_count` has no counterpart (see dh_stream_create_cu_mask). */
int dh_gemm(const void *a, const void *b, void *d, int64_t a_rows, int64_t a_cols, int64_t b_rows, int64_t b_cols,
            int transa, int transb, int accumulate, int dtype, int out_dtype, void *workspace,
            size_t workspace_bytes, void *stream);

/* The one layout dh_gemm refuses (as the reference does, "TT layout not allowed", csrc/operators/gemm.cu:3-170):
 * D [n, m] = B^T @ A^T for A [m, k] and B [k, n], both row-major.  It is the weight-gradient product dW = dY^T X
 * with X handed over transposed (A = X^T [K, T]) and dY [T, N] as it is: the cheaper of the two operands to
 * transpose when the weight has fewer inputs than outputs.  No counterpart in the reference. */
int dh_gemm_tt(const void *a, const void *b, void *d, int64_t a_rows, int64_t a_cols, int64_t b_rows, int64_t b_cols,
               int accumulate, int dtype, int out_dtype, void *workspace, size_t workspace_bytes, void *stream);

/* A stream whose kernels run only on the compute units named in `mask` (bit i of word i / 32; `words` x 32
 * bits must cover the device; with several XCDs bit i is compute unit i / n_xcd of XCD i % n_xcd).  The
 * MI355X form of the reference's libsmctrl partitioning (csrc/operators/smctrl.cpp:135-160, the `math_sm_count`
 * argument of pygemm, csrc/operators/ops.h:30): a kernel that fills every register file (the library GEMMs do)
 * keeps a later kernel of another stream from starting anywhere until its own last workgroup is placed, so a
 * small kernel that must start on time -- a collective -- gets compute units the compute streams never use.
 * `dh_stream_destroy` ends a stream created here (after its work has finished). */
int dh_stream_create_cu_mask(const uint32_t *mask, int words, void **stream_out);
int dh_stream_destroy(void *stream);

/* out[c * ld_out + r] = in[r * ld_in + c] for a [rows, cols] matrix of 16-bit elements
 * (bf16 / fp16; rows, cols and both leading dimensions multiples of 8).  Feeds the
 * weight-gradient product of the reference's GEMM operator (csrc/operators/gemm.cu:3-170 called
 * with transb: D = B^T A) with a row-major B^T, the layout the GEMM library runs fastest. */
int dh_transpose_2d(const void *in, void *out, int64_t rows, int64_t cols, int64_t ld_in,
                    int64_t ld_out, int dtype, void *stream);

/* ---- head block: word embedding, cross entropy, masked mean loss ------------------------
 * The per-rank arithmetic of the reference's vocab-parallel head; the all-reduces that join
 * the ranks (dhellam/operators/loss.py:22-24,52-56,61-66) are outside this library.
 * vocab_start = tp_rank * (rows of this rank's vocabulary slice). */

/* Cross entropy of `rows` rows of `cols` logits (pitch ld, any dtype; fp32 arithmetic):
 * dhellam/operators/loss.py:15-97.  Per row: row_max = max(x), sum_exp = sum exp(x - row_max),
 * predicted = x[target - vocab_start] - row_max (0 when the target is outside this slice),
 * loss = log(sum_exp) - predicted, with label smoothing
 * loss = (1 - s) loss - s mean(log softmax), s = label_smoothing cols / (cols - 1).
 * Optional outputs (NULL to skip): predicted, softmax (dtype of the logits, pitch ld_softmax),
 * target_mask (1 = target outside the slice), masked_target (local index, 0 where masked). */
int dh_cross_entropy_fwd(const void *logits, const int64_t *target, int64_t rows, int64_t cols,
                         int64_t ld, int64_t vocab_start, float label_smoothing, int dtype,
                         float *loss, float *row_max, float *sum_exp, float *predicted,
                         void *softmax, int64_t ld_softmax, uint8_t *target_mask,
                         int64_t *masked_target, void *stream);

/* grad = (softmax - onehot(target) (1 - s) [target inside] - s / cols) * dout[row]:
 * dhellam/operators/loss.py:99-127.  from_logits = 0: src is the softmax of the forward;
 * from_logits = 1: src is the logits and the softmax is recomputed from row_max / sum_exp
 * (nothing of size rows x cols is kept between forward and backward).  grad may be src. */
int dh_cross_entropy_bwd(const void *src, int64_t ld_src, int from_logits, const float *row_max,
                         const float *sum_exp, const int64_t *target, const float *dout,
                         int64_t rows, int64_t cols, int64_t vocab_start, float label_smoothing,
                         int dtype, void *grad, int64_t ld_grad, void *stream);

/* out[i, :] = vocab[ids[i] - vocab_start, :], zero rows for ids outside
 * [vocab_start, vocab_start + vocab_rows): dhellam/operators/embedding.py:16-39. */
int dh_embedding_fwd(const void *vocab, const int64_t *ids, int64_t n, int64_t hidden,
                     int64_t vocab_rows, int64_t vocab_start, int dtype, void *out, void *stream);

/* dvocab[v, :] += sum of dout[i, :] over the positions i with ids[i] = vocab_start + v, in
 * position order (deterministic): the gradient autograd forms in
 * dhellam/operators/embedding.py:42-49.  dvocab is fp32 or of dout's type. */
int dh_embedding_bwd(const void *dout, const int64_t *ids, int64_t n, int64_t hidden,
                     int64_t vocab_rows, int64_t vocab_start, int dtype, void *dvocab,
                     int dvocab_dtype, void *stream);

/* out[0] = scale * sum(x mask) / sum(mask), out[1] = sum(mask):
 * dhellam/operators/loss.py:131-153 with scale = loss_scale / num_microbatch. */
int dh_masked_mean_fwd(const float *x, const float *mask, int64_t n, float scale, float *out,
                       void *stream);

/* grad[i] = scale * mask[i] / mask_sum[0] (dhellam/operators/loss.py:155-164: the reference
 * backpropagates a gradient of one). */
int dh_masked_mean_bwd(const float *mask, const float *mask_sum, int64_t n, float scale,
                       float *grad, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DHELLAM_HIP_H */

#!/usr/bin/env python3
"""Benchmark of the per-rank operator hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over one batch: four micro-batches of one TP=8 /
sequence-parallel rank's share of a Llama-3.1-70B decoder layer (hidden 8192, 8 q + 1 kv
heads x 128, SwiGLU shard 3584, seq 4096, bf16), forward + backward, run by the
double-strand runtime (forward of micro-batch i+1 on one HIP stream, backward of
micro-batch i on another).  The same four micro-batches are also timed on one stream
(serial schedule) and the faster of the two is the headline value; both are printed.

Prints ONE JSON line: the headline tokens/s, per-kernel roofline figures measured live
with HIP events on the launch stream, and the CPU eager baseline (the oracle, timed on
this host's cores on a bounded sample).  Inputs are synthetic (seeded normal), resident
in HBM before the timed region.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak
def _measured():
    """Counter- and trace-derived figures kept under profiles/ (hardware counters cannot be read from inside the
    timed run): HBM bytes per launch of the attention backward, ceiling of any co-schedule of the layer's kernels."""
    try:
        with open(os.path.join(ROOT, "profiles", "measured.json")) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def _ensure_built():
    from dhellam_amd import _lib
    if not _lib.LIB_PATH.exists():
        from dhellam_amd.build import build
        build()


def time_gpu(fn, iters=20, warmup=3, stream=None, min_ms=50.0):
    """Mean ms per call of fn() measured with HIP events recorded on the stream the kernels are
    launched on.  The chip's clock follows the load of the last tens of milliseconds (a kernel timed
    right after idle or after light kernels runs 10-20 % slower than in a loop that has been going
    for a while), so a timing that covers less than ``min_ms`` counts as warm-up and is repeated with
    as many calls as fill that time."""
    stream = stream or torch.cuda.current_stream()
    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    for attempt in range(4):                              # the first pass is warm-up whatever it covers
        start.record(stream)
        for _ in range(iters):
            fn()
        end.record(stream)
        end.synchronize()
        total = start.elapsed_time(end)
        if total >= min_ms and attempt > 0:
            break
        if total < min_ms:
            iters = min(20000, int(iters * min_ms / max(total, 1e-3) * 1.2) + 1)
    return total / iters


def time_gpu_graph(fn, iters=50, min_ms=20.0):
    """Mean ms per call with ``iters`` calls captured in one HIP graph and the replays bracketed by
    HIP events on the replay stream: for kernels of a few microseconds this measures the kernels,
    not the Python launch path.  The graph is replayed for ``min_ms`` untimed (clock settled, as in
    time_gpu) and then for ``min_ms`` timed."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            for _ in range(iters):
                fn()
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record(s)
        g.replay()
        end.record(s)
        end.synchronize()
        reps = max(1, min(2000, int(min_ms / max(start.elapsed_time(end), 1e-3)) + 1))
        for _ in range(reps):
            g.replay()
        start.record(s)
        for _ in range(reps):
            g.replay()
        end.record(s)
        end.synchronize()
    torch.cuda.current_stream().wait_stream(s)
    return start.elapsed_time(end) / (iters * reps)


def kernel_rooflines(cfg):
    """Per-operator achieved rate against its roofline at the 70B-shard shapes (and the
    ring / MoE shapes).  Algorithmic work only: compulsory bytes, unmasked MACs."""
    from dhellam_amd import _Clib
    from dhellam_amd import _lib as L_
    from dhellam_amd.operators import moe
    from dhellam_amd.operators.bda import bda_fwd
    from dhellam_amd.operators.layernorm import pylayernorm_bwd, pylayernorm_fwd
    from dhellam_amd.operators.rope import rope_fwd
    from dhellam_amd.operators.swiglu import swiglu, swiglu_back
    dev, dt = "cuda", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(s, generator=g, device=dev, dtype=torch.float32).to(dt)
    res = []
    lib = L_.load()
    floors = {}

    def copy_floor_ms(work_bytes):
        """ms of the plain copy kernel (dh_copy_bytes) moving the same number of bytes (half read, half written),
        timed the same way: what this machine gives a kernel of that size that does nothing but stream."""
        n = int(work_bytes // 2) // 16 * 16
        if n not in floors:
            src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
            dst = torch.empty_like(src)
            floors[n] = time_gpu_graph(lambda: L_.check(lib.dh_copy_bytes(src.data_ptr(), dst.data_ptr(), n,
                                                                          torch.cuda.current_stream().cuda_stream)))
            del src, dst
        return floors[n]

    def add(name, bound, work, ms, unit_work):
        rate = work / (ms * 1e-3)
        if bound == "hbm":
            ach, peak, unit = rate / 1e9, HBM_PEAK_GBS, "GB/s"
        else:
            ach, peak, unit = rate / 1e12, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s"
        row = {"kernel": name, "bound": bound, "ms": round(ms, 5), "achieved": round(ach, 2), "peak": peak,
               "unit": unit, "frac": round(ach / peak, 4), "work": unit_work}
        if bound == "hbm":
            # the bar for a bandwidth kernel: 70 % of the HBM peak, or within 10 % of a plain copy of the same bytes
            fl = copy_floor_ms(work)
            row["copy_floor_ms"] = round(fl, 5)
            row["vs_copy_floor"] = round(ms / fl, 3)
            row["meets_bar"] = bool(ach / peak >= 0.70 or ms <= 1.10 * fl)
        res.append(row)

    R, H, F, T = cfg.sp_rows, cfg.hidden_size, cfg.ffn_per_rank, cfg.tokens
    hq, hk, d = cfg.heads_per_rank, cfg.groups_per_rank, cfg.head_dim
    e = 2
    # --- norm -----------------------------------------------------------------------------
    for rows in (R, 8 * R, 64 * R):
        x, gm, dy = rn(rows, H), torch.ones(H, device=dev, dtype=dt), rn(rows, H)
        y, _, rs, _ = pylayernorm_fwd(x, gm, None, 1e-5, 0, False, None)
        ms = time_gpu_graph(lambda: pylayernorm_fwd(x, gm, None, 1e-5, 0, False, None))
        add(f"rmsnorm_fwd[{rows}x{H}]", "hbm", 2 * rows * H * e + H * e + 4 * rows, ms, "2RHe+He+4R bytes")
        ms = time_gpu_graph(lambda: pylayernorm_bwd(dy, x, None, rs, gm, 0, False, None))
        add(f"rmsnorm_bwd[{rows}x{H}]", "hbm", 3 * rows * H * e + 4 * rows + 2 * H * e, ms, "3RHe+4R+2He bytes")
        del x, dy, y
    # --- rope -----------------------------------------------------------------------------
    qkv = rn(T, cfg.qkv_per_rank)
    q = qkv[:, : hq * d].view(T, hq, d)
    k = qkv[:, hq * d:(hq + hk) * d].view(T, hk, d)
    ms = time_gpu_graph(lambda: rope_fwd(q, k, None, cfg.rope_theta, cfg.seq_length, None, False, inplace=True))
    add(f"rope[{T}x({hq}+{hk})x{d}]", "hbm", 2 * T * (hq + hk) * d * e, ms, "2T(Hq+Hk)de bytes")
    # --- swiglu ---------------------------------------------------------------------------
    yy, gg = rn(T, 2 * F), rn(T, F)
    ms = time_gpu_graph(lambda: swiglu(yy))
    add(f"swiglu_fwd[{T}x{2 * F}]", "hbm", 3 * T * F * e, ms, "3TFe bytes")
    ms = time_gpu_graph(lambda: swiglu_back(gg, yy))
    add(f"swiglu_bwd[{T}x{2 * F}]", "hbm", 5 * T * F * e, ms, "5TFe bytes")
    # --- residual add -----------------------------------------------------------------------
    a, b = rn(R, H), rn(R, H)
    o = torch.empty_like(a)
    ms = time_gpu_graph(lambda: bda_fwd(a, b, out=o))
    add(f"residual_add[{R}x{H}]", "hbm", 3 * R * H * e, ms, "3RHe bytes")
    gm, so = torch.ones(H, device=dev, dtype=dt), torch.empty_like(a)
    ms = time_gpu_graph(lambda: pylayernorm_fwd(a, gm, None, 1e-5, 0, False, None, residual=b, sum_out=so))
    add(f"residual_add_rmsnorm_fwd[{R}x{H}]", "hbm", 4 * R * H * e + H * e + 4 * R, ms, "4RHe+He+4R bytes")
    del yy, gg
    # --- attention (70B shard: causal, S=4096, 8q/1kv, d=128) --------------------------------
    v = qkv[:, (hq + hk) * d:].view(T, hk, d)
    cu = torch.tensor([0, T], dtype=torch.int32, device=dev)
    sc = 1.0 / math.sqrt(d)
    fl_fwd = 4 * d * hq * (T * (T + 1) / 2)
    out_l = _Clib.pymha_varlen_fwd(q, k, v, cu, cu, T, T, 0.0, sc, True, False, 0, False)
    ms = time_gpu(lambda: _Clib.pymha_varlen_fwd(q, k, v, cu, cu, T, T, 0.0, sc, True, False, 0, False))
    add(f"attn_fwd[causal S={T} {hq}q/{hk}kv d={d}]", "mfma", fl_fwd, ms, "4*d*Hq*S(S+1)/2 flop")
    do = rn(T, hq, d)
    sp = torch.cuda.current_stream().cuda_stream
    dq, dk, dv = torch.empty_like(do), torch.empty(T, hk, d, device=dev, dtype=dt), torch.empty(T, hk, d, device=dev, dtype=dt)
    bw = lambda: _Clib._attn_bwd_raw(do, q, k, v, out_l[0], out_l[5], dq, dk, dv, None, cu, cu, T, T, sc, True, sp)
    ms_bwd = time_gpu(bw)
    add(f"attn_bwd[causal S={T} {hq}q/{hk}kv d={d}]", "mfma", 2.5 * fl_fwd, ms_bwd, "2.5 * fwd flop (delta, dK/dV keeping dS, head-split sum and dQ-from-dS kernels)")
    # --- ring step (32q/8kv, d=128, q 4096, kv chunk 4096): one causal and one full-block step -------
    hq1, hk1, S1 = 32, 8, 4096
    q1, k1, v1, do1 = rn(S1, hq1, d), rn(S1, hk1, d), rn(S1, hk1, d), rn(S1, hq1, d)
    cu1 = torch.tensor([0, S1], dtype=torch.int32, device=dev)
    cuh = torch.tensor([0, S1 // 2], dtype=torch.int32, device=dev)
    fl_half = 4 * d * hq1 * (S1 * S1 / 2)
    o1 = _Clib.pymha_varlen_fwd(q1, k1, v1, cu1, cu1, S1, S1, 0.0, sc, True, False, 0, False)
    ms = time_gpu(lambda: _Clib.pymha_varlen_fwd(q1, k1, v1, cu1, cu1, S1, S1, 0.0, sc, True, False, 0, False))
    add("ring_step_fwd[diag 32q/8kv q4096 kv4096]", "mfma", fl_half, ms, "4*d*Hq*S^2/2 flop")
    ms = time_gpu(lambda: _Clib.pymha_varlen_fwd(q1, k1[: S1 // 2], v1[: S1 // 2], cu1, cuh, S1, S1 // 2, 0.0, sc, False, False, 0, False))
    add("ring_step_fwd[lower 32q/8kv q4096 kv2048]", "mfma", fl_half, ms, "4*d*Hq*S^2/2 flop")
    dq1, dk1, dv1 = torch.empty_like(q1), torch.empty_like(k1), torch.empty_like(v1)
    ms = time_gpu(lambda: _Clib._attn_bwd_raw(do1, q1, k1, v1, o1[0], o1[5], dq1, dk1, dv1, None, cu1, cu1, S1, S1, sc, True, sp), iters=10)
    add("ring_step_bwd[diag 32q/8kv q4096 kv4096]", "mfma", 2.5 * fl_half, ms, "2.5 * fwd flop")
    # merge of 4 partial results (ring rank 3: all steps cover all rows)
    outs = [rn(S1, hq1, d) for _ in range(4)]
    lses = [torch.randn(1, hq1, S1, generator=g, device=dev) for _ in range(4)]
    om, lm = torch.empty(S1, hq1, d, device=dev, dtype=dt), torch.empty(1, hq1, S1, device=dev)
    ms = time_gpu_graph(lambda: _Clib.pyattn_merge(outs, lses, [0] * 4, [S1] * 4, om, lm))
    add("attn_merge[4 steps x 4096x32x128]", "hbm", 5 * S1 * hq1 * d * e + 5 * 4 * S1 * hq1, ms, "(n+1)THde+(n+1)4TH bytes")
    del q1, k1, v1, do1, outs, lses, om, dq1, dk1, dv1, o1
    # --- MoE: 8192 tokens, 8 experts top-2, hidden 4096, expert FFN 14336, this rank holds experts 0,1 ----
    Tm, Hm, E, K, Fm = 8192, 4096, 8, 2, 14336
    logits = torch.randn(Tm, E, generator=g, device=dev)
    xm = rn(Tm, Hm)
    idx, gates, _ = moe.route_topk(logits, K)
    plan, _ = moe.sort_assignments(idx, E)
    Rm = int(plan.expert_offsets[2].item())
    ms = time_gpu_graph(lambda: moe.permute_fwd(xm, plan, 0, 2, Rm))
    add(f"moe_permute[R={Rm} H={Hm}]", "hbm", 2 * Rm * Hm * e + 8 * Rm, ms, "2RHe+8R bytes")
    xp, _ = moe.permute_fwd(xm, plan, 0, 2, Rm)
    ms = time_gpu_graph(lambda: moe.unpermute_fwd(xp, plan, gates, 0, 2))
    add(f"moe_unpermute[R={Rm} T={Tm} H={Hm}]", "hbm", Rm * Hm * e + Tm * Hm * e + 8 * Rm, ms, "RHe+THe+8R bytes")
    w1 = (torch.randn(2, 2 * Fm, Hm, generator=g, device=dev) * 0.02).to(dt)
    w2 = (torch.randn(2, Hm, Fm, generator=g, device=dev) * 0.02).to(dt)
    offs = plan.expert_offsets[0:3]
    ms = time_gpu(lambda: moe.expert_ffn_fwd(xp, w1, w2, offs), iters=5, warmup=2)
    add(f"moe_expert_ffn_fwd[R={Rm} H={Hm} F={Fm}]", "mfma", 6.0 * Rm * Hm * Fm, ms, "6RHF flop (grouped GEMMs + SwiGLU)")
    y, saved, _ = moe.expert_ffn_fwd(xp, w1, w2, offs)
    dyp = rn(Rm, Hm)
    ms = time_gpu(lambda: moe.expert_ffn_bwd(dyp, xp, w1, w2, offs, saved), iters=5, warmup=2)
    add(f"moe_expert_ffn_bwd[R={Rm} H={Hm} F={Fm}]", "mfma", 12.0 * Rm * Hm * Fm, ms, "12RHF flop")
    # --- head block: Llama-3.1 vocabulary 128256 over TP = 8 (16032 columns), one micro-batch of 4096 tokens ----
    from dhellam_amd.common import parallel_state
    from dhellam_amd.operators.embedding import word_embedding_bwd, word_embedding_fwd
    from dhellam_amd.operators.loss import cross_entropy_bwd, cross_entropy_fwd
    from dhellam_amd import _lib as L
    Vp = 128256 // 8
    g2 = torch.Generator(device=dev).manual_seed(1)
    rn = lambda *s: torch.randn(s, generator=g2, device=dev, dtype=torch.float32).to(dt)
    parallel_state.set_tensor_model_parallel(0, 8)
    logits = (rn(T, Vp).float() * 3).to(dt)
    tgt = torch.randint(0, 128256, (T,), generator=g2, device=dev)
    ce_in = {"vocab_parallel_logits": logits, "target": tgt}
    ms = time_gpu_graph(lambda: cross_entropy_fwd(ce_in, 0.0, keep_softmax=False))
    add(f"cross_entropy_fwd[{T}x{Vp}]", "hbm", T * Vp * e + 20 * T, ms, "TVe+20T bytes (loss and row statistics only)")
    ce_out = cross_entropy_fwd(ce_in, 0.0, keep_softmax=False)
    dl, gbuf = torch.randn(T, generator=g2, device=dev), torch.empty_like(logits)
    ms = time_gpu_graph(lambda: cross_entropy_bwd([ce_in, ce_out], dl, grad_out=gbuf))
    add(f"cross_entropy_bwd[{T}x{Vp}]", "hbm", 2 * T * Vp * e + 20 * T, ms, "2TVe+20T bytes (softmax recomputed from the logits)")
    del logits, gbuf, ce_out
    table = rn(Vp, H)
    ids = torch.randint(0, 128256, (1, T), generator=g2, device=dev)
    ids[0, : T // 2] = torch.randint(0, Vp, (T // 2,), generator=g2, device=dev)   # every rank sees ~1/8 in real runs; here 9/16
    inside = int(((ids >= 0) & (ids < Vp)).sum().item())
    em_in = {"vocab": table, "token_ids": ids}
    ms = time_gpu_graph(lambda: word_embedding_fwd(em_in))
    add(f"embedding_fwd[{T}x{H}, {inside} ids inside]", "hbm", (inside + T) * H * e + 8 * T, ms, "(Tin+T)He+8T bytes")
    table.main_grad = torch.zeros(Vp, H, device=dev, dtype=torch.float32)
    dh_ = rn(1, T, H)
    em_out = word_embedding_fwd(em_in)
    ms = time_gpu_graph(lambda: word_embedding_bwd([em_in, em_out], dh_))
    add(f"embedding_bwd[{T}x{H}, {inside} ids inside]", "hbm", inside * H * (e + 8) + 8 * T, ms, "Tin*H(e+8)+8T bytes (fp32 main_grad read+write)")
    # the whole head: final norm -> logits GEMM -> cross entropy -> masked mean, and back (GEMM-dominated)
    from dhellam_amd.core import dshb
    hid = rn(T, 1, H)
    gam = torch.ones(H, device=dev, dtype=dt)
    labels = torch.randint(0, 128256, (1, T), generator=g2, device=dev)
    lmask = torch.ones(1, T, device=dev, dtype=torch.int64)
    gam.main_grad = torch.zeros_like(gam)

    from dhellam_amd._Clib import keep_transposed as _keep_t
    _keep_t(table)                             # as DSHB / DSLLMStep hold it: the logits product's data gradient runs against W^T
    def head_step():
        _, hctx = dshb.post_process(hid, gam, None, labels, lmask, table, 4, 1.0)
        dshb.post_process_bwd(hctx)
    ms = time_gpu(head_step, iters=5, warmup=2)
    add(f"head_block_fwd_bwd[{T}x{H} -> {Vp}]", "mfma", 6.0 * T * H * Vp, ms, "6THV flop (logits GEMM fwd, dgrad, wgrad; norm, cross entropy, loss around them)")
    parallel_state.set_tensor_model_parallel(0, 1)
    del table, dh_, em_out, hid
    # --- the layer's twelve dense products (library kernels through dh_gemm), as the layer calls them -------
    from dhellam_amd._Clib import keep_transposed
    from dhellam_amd.operators.layernorm_column import dgrad_bwd, gemm_fwd, wgrad_bwd
    for name, n_out, k_in in (("qkv", cfg.qkv_per_rank, H), ("attn_out", H, hq * d), ("fc1", 2 * F, H), ("fc2", H, F)):
        x, w, dy = rn(T, k_in), rn(n_out, k_in), rn(T, n_out)
        keep_transposed(w)                      # as the layer holds its weights: dgrad runs against W^T
        dw = torch.zeros(n_out, k_in, device=dev, dtype=dt)
        flop = 2.0 * T * n_out * k_in
        for what, fn in (("fwd", lambda: gemm_fwd(None, x, w, None, "TN", False, 0, True, None)),
                         ("dgrad", lambda: dgrad_bwd(None, dy, w, None, "NN", False, 0, True, None)),
                         ("wgrad", lambda: wgrad_bwd(None, dy, x, dw, True, "NT", False, 0, True, None))):
            add(f"dense_gemm[{name} {what} T={T} N={n_out} K={k_in}]", "mfma", flop, time_gpu(fn, iters=10, warmup=3),
                "2TNK flop (hipBLASLt through dh_gemm; dgrad against the resident W^T; wgrad includes the transpose of dY where it is used)")
        del x, w, dy, dw
    return res


def _median_s(fn, reps: int = 3, warmup: int = 1) -> float:
    for _ in range(warmup):
        fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[len(ts) // 2]


def _oracle_cfg(cfg):
    return dict(hidden=cfg.hidden_size, heads=cfg.heads_per_rank, groups=cfg.groups_per_rank, head_dim=cfg.head_dim,
                ffn=cfg.ffn_per_rank, seq=cfg.seq_length, batch=cfg.micro_batch_size,
                tp=cfg.tensor_model_parallel_size, tp_rank=cfg.tp_rank, eps=cfg.layernorm_epsilon, theta=cfg.rope_theta)


def cpu_baseline(cfg):
    """The oracle's eager PyTorch path on this host's cores (the reference's own operators cannot run without a GPU:
    every wrapper enters a CUDA stream), 1 warm-up + 3 timed repetitions, median, same seeded inputs as the GPU run.
    The headline entry is ONE micro-batch of the 70B-shard layer at full shape (fp32, forward + backward by autograd);
    ``others`` holds the fp32 parity layer at full shape, the MoE rank share's index / row-move operators at full
    shape, and bounded, LABELLED samples of the two heavy ones (expert FFN: 512 of the ~4100 rows; ring attention:
    one diagonal step of 4 of the 32 query heads), each with the figure scaled to the full size."""
    import numpy as np
    from dhellam_amd.core.layer import make_microbatch, make_weights, small_fp32_layer
    from oracle import attention as OA
    from oracle import layer as OL
    from oracle import moe as OM
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    w = {k: v for k, v in make_weights(cfg, 0, device="cpu").items() if v.is_floating_point()}
    mb = make_microbatch(cfg, 0, device="cpu")
    oc = _oracle_cfg(cfg)
    t = _median_s(lambda: OL.layer_fwd_bwd(oc, w, mb, dtype=torch.float32))
    others = []
    # the fp32 parity layer (hidden 1024, 16 x 64 MHA, FFN 2816, batch 2 x seq 512), full shape
    c0 = small_fp32_layer()
    w0 = {k: v for k, v in make_weights(c0, 0, device="cpu").items() if v.is_floating_point()}
    mb0 = make_microbatch(c0, 0, device="cpu")
    t0 = _median_s(lambda: OL.layer_fwd_bwd(_oracle_cfg(c0), w0, mb0, dtype=torch.float32))
    others.append({"what": "fp32 parity layer fwd+bwd (hidden 1024, 16x64 MHA, FFN 2816, 2x512 tokens), full shape",
                   "ms": round(t0 * 1e3, 1), "tokens_per_s": round(c0.tokens / t0, 1), "scaled": False})
    # MoE rank share: 8192 tokens, 8 experts, top-2, hidden 4096; route + sort, permute, unpermute at full shape
    g = torch.Generator().manual_seed(0)
    Tm, Hm, E, K, Fm = 8192, 4096, 8, 2, 14336
    logits = torch.randn(Tm, E, generator=g).numpy()
    xm = torch.randn(Tm, Hm, generator=g).to(torch.bfloat16)
    idx, gates = OM.route_topk(logits, K)
    tpe, offs, sidx, dest = OM.sort_assignments(idx, E)
    t_route = _median_s(lambda: OM.sort_assignments(OM.route_topk(logits, K)[0], E))
    t_perm = _median_s(lambda: OM.permute(xm, sidx, offs, 0, 2, K, dtype=torch.bfloat16))
    xp = OM.permute(xm, sidx, offs, 0, 2, K, dtype=torch.bfloat16)
    gt = torch.from_numpy(np.asarray(gates, dtype=np.float32))
    t_unp = _median_s(lambda: OM.unpermute(xp, dest, offs, 0, 2, Tm, K, gates=gt, dtype=torch.float32))
    R = int(offs[2] - offs[0])
    others.append({"what": f"MoE route_topk + sort ({Tm} tokens x {E} experts, top-{K}), full shape",
                   "ms": round(t_route * 1e3, 2), "scaled": False})
    others.append({"what": f"MoE permute (R={R} rows x {Hm}, bf16), full shape", "ms": round(t_perm * 1e3, 2),
                   "GB_per_s": round((2 * R * Hm * 2 + 8 * R) / t_perm / 1e9, 2), "scaled": False})
    others.append({"what": f"MoE unpermute with gates (R={R} -> {Tm} tokens x {Hm}), full shape",
                   "ms": round(t_unp * 1e3, 2), "GB_per_s": round((R * Hm * 2 + Tm * Hm * 2 + 8 * R) / t_unp / 1e9, 2),
                   "scaled": False})
    # expert FFN fwd+bwd on a sample of 512 rows (256 per expert), fp32, scaled by rows
    rs = 512
    w1 = torch.randn(2, 2 * Fm, Hm, generator=g) * 0.02
    w2 = torch.randn(2, Hm, Fm, generator=g) * 0.02
    xs = torch.randn(rs, Hm, generator=g, requires_grad=True)
    so = np.array([0, rs // 2, rs])

    def ffn():
        y, _, _ = OM.grouped_ffn(xs, w1.requires_grad_(), w2.requires_grad_(), so, dtype=torch.float32)
        y.sum().backward()
    t_ffn = _median_s(ffn)
    others.append({"what": f"MoE expert FFN fwd+bwd (2 experts, H {Hm}, F {Fm}): {rs} of {R} rows timed, SCALED to {R} rows",
                   "ms": round(t_ffn * 1e3 * R / rs, 1), "sample_ms": round(t_ffn * 1e3, 1),
                   "TFLOP_per_s": round(18.0 * rs * Hm * Fm / t_ffn / 1e12, 3), "scaled": True})
    del w1, w2
    # ring attention: one diagonal (causal 4096 x 4096) step, 4 of the 32 query heads on 1 of the 8 kv heads, fwd + bwd
    S, hq, hk, d = 4096, 4, 1, 128
    q, k, v, do = (torch.randn(S, h, d, generator=g) for h in (hq, hk, hk, hq))
    cu = torch.tensor([0, S], dtype=torch.int32)

    def ring_step():
        o, l = OA.attn_fwd(q, k, v, cu, cu, d ** -0.5, True, torch.float32)
        OA.attn_bwd(do, q, k, v, o, l, cu, cu, d ** -0.5, True, torch.float32)
    t_ring = _median_s(ring_step, reps=3, warmup=1)
    others.append({"what": "ring attention step fwd+bwd (diagonal, q 4096 x kv 4096, d 128): 4 of 32 query heads timed, "
                           "SCALED to 32 heads x 4 steps",
                   "ms": round(t_ring * 1e3 * 8 * 4, 1), "sample_ms": round(t_ring * 1e3, 1), "scaled": True})
    return {"value": round(cfg.tokens / t, 1), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "ms_per_microbatch": round(t * 1e3, 1),
            "sample": f"median of 3 reps after 1 warm-up of ONE micro-batch ({cfg.tokens} tokens) of the same layer, "
                      f"full shape, fp32 eager PyTorch + autograd on the host (the oracle)",
            "others": others}


def profile_op(name: str, iters: int = 5):
    """Run one operator a few times and exit (target of `rocprofv3 --pmc ... -- python bench.py
    --profile-op NAME`).  ``copy`` is the calibration kernel: a 1 GiB device-to-device copy whose
    fetch and write sizes are known."""
    from dhellam_amd import _Clib, _lib
    dev, dt = "cuda", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(s, generator=g, device=dev, dtype=torch.float32).to(dt)
    if name == "copy":
        n = 1 << 30
        a = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
        b = torch.empty_like(a)
        lib = _lib.load()
        fn = lambda: _lib.check(lib.dh_copy_bytes(a.data_ptr(), b.data_ptr(), n, torch.cuda.current_stream().cuda_stream))
    elif name in ("attn_fwd", "attn_bwd", "ring_fwd", "ring_bwd"):
        T, hq, hk, d = (4096, 8, 1, 128) if name.startswith("attn") else (4096, 32, 8, 128)
        q, k, v, do = rn(T, hq, d), rn(T, hk, d), rn(T, hk, d), rn(T, hq, d)
        cu = torch.tensor([0, T], dtype=torch.int32, device=dev)
        sc = 1.0 / math.sqrt(d)
        o = _Clib.pymha_varlen_fwd(q, k, v, cu, cu, T, T, 0.0, sc, True, False, 0, False)
        if name.endswith("fwd"):
            fn = lambda: _Clib.pymha_varlen_fwd(q, k, v, cu, cu, T, T, 0.0, sc, True, False, 0, False)
        else:
            dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
            sp = torch.cuda.current_stream().cuda_stream
            fn = lambda: _Clib._attn_bwd_raw(do, q, k, v, o[0], o[5], dq, dk, dv, None, cu, cu, T, T, sc, True, sp)
    elif name in ("moe_ffn_fwd", "moe_ffn_bwd"):
        from dhellam_amd.operators import moe
        Tm, Hm, E, K, Fm = 8192, 4096, 8, 2, 14336
        logits = torch.randn(Tm, E, generator=g, device=dev)
        xm = rn(Tm, Hm)
        idx, gates, _ = moe.route_topk(logits, K)
        plan, _ = moe.sort_assignments(idx, E)
        Rm = int(plan.expert_offsets[2].item())
        xp, _ = moe.permute_fwd(xm, plan, 0, 2, Rm)
        w1 = (torch.randn(2, 2 * Fm, Hm, generator=g, device=dev) * 0.02).to(dt)
        w2 = (torch.randn(2, Hm, Fm, generator=g, device=dev) * 0.02).to(dt)
        offs = plan.expert_offsets[0:3]
        if name.endswith("fwd"):
            fn = lambda: moe.expert_ffn_fwd(xp, w1, w2, offs)
        else:
            y, saved, _ = moe.expert_ffn_fwd(xp, w1, w2, offs)
            dyp = rn(Rm, Hm)
            fn = lambda: moe.expert_ffn_bwd(dyp, xp, w1, w2, offs, saved)
    elif name in ("norm", "swiglu", "swiglu_t", "cross_entropy", "transpose"):
        # bandwidth kernels at sizes beyond the 256 MB last-level cache (norm, SwiGLU) / at the head-block and
        # weight-gradient shapes (cross entropy, transpose); forward then backward in each iteration
        from dhellam_amd.operators.layernorm import pylayernorm_bwd, pylayernorm_fwd
        from dhellam_amd.operators.loss import cross_entropy_bwd, cross_entropy_fwd
        from dhellam_amd.operators.swiglu import swiglu, swiglu_back
        if name == "norm":
            x, gm, dy = rn(32768, 8192), torch.ones(8192, device=dev, dtype=dt), rn(32768, 8192)
            _, _, rs, _ = pylayernorm_fwd(x, gm, None, 1e-5, 0, False, None)
            fn = lambda: (pylayernorm_fwd(x, gm, None, 1e-5, 0, False, None), pylayernorm_bwd(dy, x, None, rs, gm, 0, False, None))
        elif name == "swiglu":
            yy, gg = rn(16384, 7168), rn(16384, 3584)
            fn = lambda: (swiglu(yy), swiglu_back(gg, yy))
        elif name == "swiglu_t":       # the kernels that write their result transposed as well
            yy, gg = rn(16384, 7168), rn(16384, 3584)
            fn = lambda: (swiglu(yy, with_transposed=True), swiglu_back(gg, yy, with_transposed=True))
        elif name == "cross_entropy":
            lg = rn(4096, 16032)
            ce_in = {"vocab_parallel_logits": lg, "target": torch.randint(0, 16032, (4096,), generator=g, device=dev)}
            dl, gbuf = torch.ones(4096, device=dev), torch.empty_like(lg)
            fn = lambda: cross_entropy_bwd([ce_in, cross_entropy_fwd(ce_in, 0.0, keep_softmax=False)], dl, grad_out=gbuf)
        else:
            src, dst = rn(4096, 8192), torch.empty(8192, 4096, device=dev, dtype=dt)
            fn = lambda: _Clib.transpose_2d(src, dst)
    elif name in ("rope", "residual_add", "add_norm", "norm_shard", "merge", "permute", "unpermute", "copy_shard"):
        # the bandwidth kernels at the configurations' own shapes (70B shard: 512 x 8192 norm rows, 4096 tokens of
        # 8 q + 1 kv heads; ring: 4 steps of 4096 x 32 x 128; MoE: 8192 tokens, hidden 4096, this rank's 2 experts)
        from dhellam_amd.operators import moe
        from dhellam_amd.operators.bda import bda_fwd
        from dhellam_amd.operators.layernorm import pylayernorm_bwd, pylayernorm_fwd
        from dhellam_amd.operators.rope import rope_fwd
        if name == "rope":
            qkv = rn(4096, 1280)
            q, k = qkv[:, :1024].view(4096, 8, 128), qkv[:, 1024:1152].view(4096, 1, 128)
            fn = lambda: rope_fwd(q, k, None, 500000.0, 4096, None, False, inplace=True)
        elif name == "residual_add":
            a, b = rn(512, 8192), rn(512, 8192)
            o = torch.empty_like(a)
            fn = lambda: bda_fwd(a, b, out=o)
        elif name == "add_norm":
            a, b, gm = rn(512, 8192), rn(512, 8192), torch.ones(8192, device=dev, dtype=dt)
            so = torch.empty_like(a)
            fn = lambda: pylayernorm_fwd(a, gm, None, 1e-5, 0, False, None, residual=b, sum_out=so)
        elif name == "norm_shard":
            x, gm, dy = rn(512, 8192), torch.ones(8192, device=dev, dtype=dt), rn(512, 8192)
            _, _, rs, _ = pylayernorm_fwd(x, gm, None, 1e-5, 0, False, None)
            fn = lambda: (pylayernorm_fwd(x, gm, None, 1e-5, 0, False, None), pylayernorm_bwd(dy, x, None, rs, gm, 0, False, None))
        elif name == "copy_shard":      # the plain copy kernel on the norm's bytes: 8 MiB read, 8 MiB written
            n = 512 * 8192 * 2
            a = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
            b = torch.empty_like(a)
            lib = _lib.load()
            fn = lambda: _lib.check(lib.dh_copy_bytes(a.data_ptr(), b.data_ptr(), n, torch.cuda.current_stream().cuda_stream))
        elif name == "merge":
            outs = [rn(4096, 32, 128) for _ in range(4)]
            lses = [torch.randn(1, 32, 4096, generator=g, device=dev) for _ in range(4)]
            om, lm = torch.empty(4096, 32, 128, device=dev, dtype=dt), torch.empty(1, 32, 4096, device=dev)
            fn = lambda: _Clib.pyattn_merge(outs, lses, [0] * 4, [4096] * 4, om, lm)
        else:
            Tm, Hm, E, K = 8192, 4096, 8, 2
            logits = torch.randn(Tm, E, generator=g, device=dev)
            xm = rn(Tm, Hm)
            idx, gates, _ = moe.route_topk(logits, K)
            plan, _ = moe.sort_assignments(idx, E)
            Rm = int(plan.expert_offsets[2].item())
            xp, _ = moe.permute_fwd(xm, plan, 0, 2, Rm)
            print(f"moe rows of this rank: {Rm}", flush=True)
            fn = (lambda: moe.permute_fwd(xm, plan, 0, 2, Rm)) if name == "permute" else (lambda: moe.unpermute_fwd(xp, plan, gates, 0, 2))
    elif name in ("gg_nt", "gemm_nt"):
        # one [4096, 8192] x [7168, 8192]^T product: the grouped GEMM kernel (two groups of 2048 rows, full tiles
        # only) and the library GEMM of the same shape, for side-by-side counter runs
        from dhellam_amd.operators import moe
        R, N, K = 4096, 7168, 8192
        a, c = rn(R, K), torch.empty(R, N, device=dev, dtype=dt)
        if name == "gg_nt":
            b = (torch.randn(2, N, K, generator=g, device=dev) * 0.02).to(dt)
            offs = torch.tensor([0, 2048, 4096], dtype=torch.int32, device=dev)
            fn = lambda: moe.grouped_gemm_nt(a, b, offs, out=c)
        else:
            b = (torch.randn(N, K, generator=g, device=dev) * 0.02).to(dt)
            from dhellam_amd._Clib import dense_gemm
            fn = lambda: dense_gemm(b, a, c, True, False, False)     # the library kernel through dh_gemm
    elif name == "layer":
        # the serial schedule alone: four micro-batches of the 70B-shard layer, forward + backward
        from dhellam_amd.core.layer import LayerRunner, llama70b_tp8_shard, make_microbatch, make_weights
        cfg = llama70b_tp8_shard()
        runner = LayerRunner(cfg, make_weights(cfg, 0, gen_device="cuda"))
        mbs = [make_microbatch(cfg, i, gen_device="cuda") for i in range(4)]
        fn = lambda: runner.run_serial(mbs)
    else:
        raise SystemExit(f"unknown --profile-op {name}")
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()


def analyze_trace(path: str, cus: int = 256, lds_per_cu: int = 160 * 1024, regs_per_simd: int = 512,
                  max_waves_per_simd: int = 8) -> str:
    """Overlap headroom of the SERIAL schedule from a `rocprofv3 --kernel-trace --output-format csv` trace of
    `bench.py --profile-op layer` (no GPU needed): how much compute-unit time one step leaves unused, i.e. the most
    any co-schedule of a second strand could fill.  Per kernel: workgroups, how many fit the GPU at once (limited
    by LDS, registers and wave slots), rounds, and the share of its CU-time that the last, partly filled round
    leaves idle (compute units without any workgroup); plus the gaps between consecutive kernels on the stream.
    All workgroups of a kernel are taken to run equally long.  Returns a markdown report."""
    import csv
    import re
    rows = []
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            rows.append(r)
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    first = next(i for i, r in enumerate(rows) if "norm_fwd_kernel" in r["Kernel_Name"])
    layer = rows[first:]
    per_iter = len(layer) // 5                   # --profile-op runs the step five times
    win = layer[-per_iter:]
    span = int(win[-1]["End_Timestamp"]) - int(win[0]["Start_Timestamp"])
    busy = sum(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]) for r in win)

    def short(name):
        name = re.sub(r"\(.*", "", name)
        name = re.sub(r"<.*", "", name)
        name = name.replace("void ", "").replace("dh::", "")
        m = re.match(r"_ZN2dh(\d+)(\w+)", name)
        if m:
            name = m.group(2)[: int(m.group(1))]
        return name[:44]

    agg = {}
    idle_tail = 0.0
    for r in win:
        dur = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
        wg = int(r["Workgroup_Size_X"]) * int(r["Workgroup_Size_Y"]) * int(r["Workgroup_Size_Z"])
        grid = int(r["Grid_Size_X"]) * int(r["Grid_Size_Y"]) * int(r["Grid_Size_Z"])
        n_wg = max(1, grid // max(wg, 1))
        waves = max(1, (wg + 63) // 64)
        regs = max(8, int(r["VGPR_Count"]) + int(r["Accum_VGPR_Count"]))
        per_simd = max(1, min(max_waves_per_simd, regs_per_simd // regs))
        fit = max(1, (per_simd * 4) // waves)
        lds = int(r["LDS_Block_Size"])
        if lds > 0:
            fit = max(1, min(fit, lds_per_cu // lds))
        cap = fit * cus
        rounds = -(-n_wg // cap)
        # a compute unit counts as busy while it holds at least one workgroup (workgroups of the last round spread
        # one per compute unit first): slots a resident workgroup leaves free on its own compute unit are not idle
        # time a second strand could have, because the resident kernel already owns that unit's pipes
        last = n_wg - (rounds - 1) * cap
        fill = ((rounds - 1) + min(last, cus) / cus) / rounds
        idle_tail += dur * (1.0 - fill)
        a = agg.setdefault(short(r["Kernel_Name"]), dict(calls=0, ns=0, idle=0.0, wgs=set(), fit=set(), rounds=set()))
        a["calls"] += 1
        a["ns"] += dur
        a["idle"] += dur * (1.0 - fill)
        a["wgs"].add(n_wg)
        a["fit"].add(fit)
        a["rounds"].add(rounds)
    gaps = span - busy
    headroom = (gaps + idle_tail) / span
    out = ["| kernel | calls | total us | share of step | workgroups | fit per CU | rounds | idle share of its CU-time |",
           "|---|---|---|---|---|---|---|---|"]
    fmt = lambda s_: "/".join(str(x) for x in sorted(s_)[:4]) + ("/.." if len(s_) > 4 else "")
    for name, a in sorted(agg.items(), key=lambda kv: -kv[1]["ns"]):
        out.append(f"| {name} | {a['calls']} | {a['ns'] / 1e3:.1f} | {a['ns'] / span:.3f} | {fmt(a['wgs'])} | {fmt(a['fit'])} | "
                   f"{fmt(a['rounds'])} | {a['idle'] / max(a['ns'], 1):.3f} |")
    out.append("")
    out.append(f"step (4 micro-batches, serial): {span / 1e6:.3f} ms; kernels busy {busy / 1e6:.3f} ms; gaps between kernels "
               f"{gaps / 1e6:.3f} ms ({gaps / span:.3f}); CU-time idle in partly filled rounds {idle_tail / 1e6:.3f} ms "
               f"({idle_tail / span:.3f})")
    out.append(f"idle CU-time / CU-time = {headroom:.3f}  ->  no co-schedule of the same kernels can be faster than "
               f"{1.0 / (1.0 - headroom):.3f}x the serial schedule")
    return "\n".join(out)


def _device_info():
    """Name, architecture, CU count and HBM size as the runtime reports them."""
    p = torch.cuda.get_device_properties(0)
    info = {"name": p.name, "arch": getattr(p, "gcnArchName", ""), "compute_units": p.multi_processor_count,
            "hbm_gib": round(p.total_memory / 2**30, 1)}
    return info


def _pick_plan(arg):
    """(plan path or None, where it came from, whether the strands enter each block together): the plan that
    ``python -m dhellam_amd.search.run`` emitted (its execute stage replays the DP's candidates and the built-in
    plan and keeps the measured winner) unless ``--plan`` says otherwise."""
    root = os.path.dirname(os.path.abspath(__file__))
    emitted = os.path.join(root, "dhellam_amd", "search", "config", "best.json")
    report = os.path.join(root, "dhellam_amd", "search", "config", "execute_report.json")
    if arg == "builtin":
        return None, "built-in plan (forced)", False
    if arg:
        return arg, f"--plan {arg}", False
    if os.path.exists(emitted):
        best = {}
        if os.path.exists(report):
            with open(report) as f:
                best = json.load(f).get("best", {})
        return emitted, (f"dhellam_amd/search/config/best.json (emitted by search + execute; winner "
                         f"{best.get('name', '?')})"), bool(best.get("lockstep_blocks", False))
    return None, "built-in plan (no emitted plan in the tree)", False


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--micro-batches", type=int, default=4)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel roofline section")
    ap.add_argument("--emulate-comm-us", type=float, default=55.0,
                    help="also time both schedules with each sequence-parallel stand-in taking this long (0: skip)")
    ap.add_argument("--plan", default=None,
                    help="plan JSON for the double-strand schedule; default: the plan the search's execute stage "
                         "emitted (dhellam_amd/search/config/best.json) when there is one, else the built-in plan; "
                         "'builtin' forces the built-in plan")
    ap.add_argument("--profile-iters", type=int, default=5,
                    help="launches of --profile-op (a few hundred put a kernel trace's average at the settled clock)")
    ap.add_argument("--profile-op", default=None,
                    help="run only this operator a few times (attn_fwd, attn_bwd, ring_fwd, ring_bwd, moe_ffn_fwd, moe_ffn_bwd, norm, swiglu, swiglu_t, cross_entropy, transpose, rope, residual_add, add_norm, norm_shard, merge, permute, unpermute, copy_shard, gg_nt, gemm_nt, layer, copy) and exit")
    ap.add_argument("--analyze-trace", default=None,
                    help="kernel-trace CSV of `rocprofv3 --kernel-trace -- python bench.py --profile-op layer`: print the "
                         "overlap headroom of the serial schedule and exit (no GPU needed)")
    args = ap.parse_args()
    if args.analyze_trace:
        print(analyze_trace(args.analyze_trace))
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures ONE GPU (one rank's share of the layer, no collectives); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    _ensure_built()
    if args.profile_op:
        torch.cuda.set_device(0)
        profile_op(args.profile_op, args.profile_iters)
        return
    from dhellam_amd.core.layer import LayerRunner, llama70b_tp8_shard, make_microbatch, make_weights
    torch.cuda.set_device(0)
    cfg = llama70b_tp8_shard()
    w = make_weights(cfg, 0, gen_device="cuda")
    mbs = [make_microbatch(cfg, i, gen_device="cuda") for i in range(args.micro_batches)]
    plan, plan_source, plan_lockstep = _pick_plan(args.plan)
    if plan_lockstep:
        import dataclasses
        cfg = dataclasses.replace(cfg, lockstep_blocks=True)
    runner = LayerRunner(cfg, w, plan=plan)
    tokens_per_step = cfg.tokens * len(mbs)

    def timed(fn, runner=runner):
        # A step is what lies between two optimizer steps: the weights have just changed, so their resident
        # transposes (used by the data-gradient GEMMs) are rebuilt inside the timed region, once per step
        # (run_serial / run_double_strand do it on entry).
        for _ in range(args.warmup):
            fn(mbs)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn(mbs)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3

    ms_serial = timed(runner.run_serial)
    ms_double = timed(runner.run_double_strand)
    best_ms, schedule = (ms_double, "double-strand") if ms_double <= ms_serial else (ms_serial, "serial")
    # The same two schedules with every sequence-parallel stand-in ALSO occupying its stream for the time the
    # collective it replaces would take (a one-wavefront delay kernel, no data moved): what the double strand is
    # for.  Reported beside the real numbers, never part of `value`.
    emulated = None
    if args.emulate_comm_us > 0:
        import dataclasses
        runner_c = LayerRunner(dataclasses.replace(cfg, comm_standin_us=args.emulate_comm_us), w, plan=plan)
        ser_c, dbl_c = timed(runner_c.run_serial, runner_c), timed(runner_c.run_double_strand, runner_c)
        runner_l = LayerRunner(dataclasses.replace(cfg, comm_standin_us=args.emulate_comm_us, lockstep_blocks=True), w,
                               plan=plan)
        dbl_l = timed(runner_l.run_double_strand, runner_l)
        emulated = {"standin_us_per_collective": args.emulate_comm_us, "collectives_per_microbatch": 8,
                    "serial_ms": round(ser_c, 4), "double_strand_ms": round(dbl_c, 4),
                    "double_strand_lockstep_ms": round(dbl_l, 4),
                    "double_strand_speedup": round(ser_c / min(dbl_c, dbl_l), 4),
                    # what one stand-in adds to the serial schedule
                    "serial_cost_us_per_standin": round((ser_c - ms_serial) * 1e3 / (8 * len(mbs)), 1)}
        # The same with stand-ins that need no compute unit (a host function of the stream: a transfer carried by a
        # copy engine or a network adapter).  Its cost to a stream includes the runtime's hand-over to a host
        # thread and back, so both costs are reported: per stand-in in the serial schedule and in the double strand.
        host = dataclasses.replace(cfg, comm_standin_us=args.emulate_comm_us, comm_standin_engine="host")
        runner_h = LayerRunner(host, w, plan=plan)
        ser_h, dbl_h = timed(runner_h.run_serial, runner_h), timed(runner_h.run_double_strand, runner_h)
        n_standins = 8 * len(mbs)
        emulated["host_function_standins"] = {
            "serial_ms": round(ser_h, 4), "double_strand_ms": round(dbl_h, 4),
            "double_strand_speedup": round(ser_h / dbl_h, 4),
            "serial_cost_us_per_standin": round((ser_h - ms_serial) * 1e3 / n_standins, 1),
            "double_strand_cost_us_per_standin": round((dbl_h - ms_double) * 1e3 / n_standins, 1)}
        # ... and with the stand-ins carried out by the resident communication proxy: one kernel per step with a
        # wavefront per strand, requests posted and waited for through the command processor (no kernel launch per
        # collective, so a request does not queue behind the other strand's GEMM).  The proxy's own log gives how long
        # each collective took on the device.
        prox = dataclasses.replace(cfg, comm_standin_us=args.emulate_comm_us, comm_standin_engine="proxy")
        runner_p = LayerRunner(prox, w, plan=plan)
        ser_p, dbl_p = timed(runner_p.run_serial, runner_p), timed(runner_p.run_double_strand, runner_p)
        durs = sorted(b - a for slot in (0, 1) for a, b in runner_p.proxy.log(slot))
        emulated["resident_proxy_standins"] = {
            "serial_ms": round(ser_p, 4), "double_strand_ms": round(dbl_p, 4),
            "double_strand_speedup": round(ser_p / dbl_p, 4),
            "serial_cost_us_per_standin": round((ser_p - ms_serial) * 1e3 / n_standins, 1),
            "double_strand_cost_us_per_standin": round((dbl_p - ms_double) * 1e3 / n_standins, 1),
            "standin_us_on_device": {"requested": args.emulate_comm_us, "median": round(durs[len(durs) // 2], 1),
                                     "max": round(durs[-1], 1), "count_last_step": len(durs)} if durs else None}
    layer_flop = 2748.8e9 * len(mbs)   # GEMM 2628.5 + attention 120.3 GFLOP per 4096-token micro-batch

    measured = _measured()
    kernels = [] if args.no_kernels else kernel_rooflines(cfg)
    dom = next((k for k in kernels if k["kernel"].startswith("attn_bwd")), None)
    roofline = None
    if dom is not None:
        # HBM bytes per launch of the backward (its four kernels), from two rocprofv3 --pmc runs
        # (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000: factors from the 1 GiB copy kernel) at this exact shape.
        roofline = {"kernel": dom["kernel"], "bound": "mfma", "achieved": dom["achieved"], "peak": dom["peak"],
                    "unit": dom["unit"], "frac": dom["frac"],
                    "traffic": measured.get("attn_bwd_70b_shard_hbm_traffic_bytes"),
                    "traffic_unit": "bytes/launch (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE, calibrated; profiles/measured.json)"}
    cpu = None if args.no_cpu_baseline else cpu_baseline(cfg)

    line = {
        "metric": "layer fwd+bwd tokens/s on 1 GPU (70B TP-shard); attn MFMA %; norm HBM GB/s",
        "value": round(tokens_per_step / (best_ms * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(best_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "Llama-3.1-70B TP=8/SP rank share of one decoder layer fwd+bwd: hidden 8192, 8q+1kv "
                               "heads x128, SwiGLU shard 3584, seq 4096, SP rows 512, RoPE theta 5e5; "
                               f"{len(mbs)} micro-batches per step", "schedule": schedule,
                   "tokens_per_step": tokens_per_step, "plan_source": plan_source,
                   # serial / double-strand / ceiling, and the same with stand-in collectives (also under
                   # "schedules" and "schedules_with_emulated_collectives" below)
                   "schedule_detail": {"serial_ms": round(ms_serial, 4), "double_strand_ms": round(ms_double, 4),
                                       "double_strand_speedup": round(ms_serial / ms_double, 4),
                                       "double_strand_ceiling": measured.get("double_strand_ceiling"),
                                       "with_emulated_collectives": emulated}},
        "schedules": {"serial_ms": round(ms_serial, 4), "double_strand_ms": round(ms_double, 4),
                      "double_strand_speedup": round(ms_serial / ms_double, 4),
                      # what ANY co-schedule of these kernels could reach: idle compute-unit time of the serial trace
                      "double_strand_ceiling": measured.get("double_strand_ceiling")},
        "schedules_with_emulated_collectives": emulated,
        "layer_mfma_frac": round(layer_flop / (best_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "device": _device_info(),
        "kernels": kernels,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

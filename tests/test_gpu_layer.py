"""GPU parity of the whole decoder layer (forward + backward through the double-strand
runtime) against the autograd oracle, and identity of the serial and double-strand
schedules."""
import pytest
import torch

from oracle import layer as OL
from tests.util import assert_close, rel_err

# Bound on the distance between a 16-bit run of the whole layer and the oracle that keeps every intermediate exact
# (fp64 / fp32): each of the ~12 tensors stored on the way carries a relative rounding error of up to 2^-9 (bf16),
# and they add up roughly in quadrature through forward and backward.
UNROUNDED_BOUND = {torch.bfloat16: 2e-2, torch.float16: 3e-3}    # measured: 2.5e-3 .. 1.3e-2 (bf16)

pytestmark = pytest.mark.gpu

GRAD_KEYS = ["ln_attn_weight", "ln_mlp_weight", "column_attn_weight", "linear_attn_weight", "column_mlp_weight",
             "linear_mlp_weight"]


def _oracle_cfg(cfg):
    return dict(hidden=cfg.hidden_size, heads=cfg.heads_per_rank, groups=cfg.groups_per_rank, head_dim=cfg.head_dim,
                ffn=cfg.ffn_per_rank, seq=cfg.seq_length, batch=cfg.micro_batch_size,
                tp=cfg.tensor_model_parallel_size, tp_rank=cfg.tp_rank, eps=cfg.layernorm_epsilon,
                theta=cfg.rope_theta, cp=cfg.context_parallel_size, cp_rank=cfg.cp_rank)


def _cpu(d):
    out = {k: v.detach().cpu() for k, v in d.items() if isinstance(v, torch.Tensor) and v.is_floating_point()}
    out.update({k: [t.detach().cpu() for t in v] for k, v in d.items() if isinstance(v, list)})
    return out


def _check_layer(cfg, oracle_dtype, round_to=None):
    from dhellam_amd.core.layer import LayerRunner, make_microbatch, make_weights
    w = make_weights(cfg, 0)
    mb = make_microbatch(cfg, 0)
    w_cpu, mb_cpu = _cpu(w), _cpu(mb)           # before the run: the gather stand-in writes into the peer buffers
    runner = LayerRunner(cfg, w)
    outs, dxs = runner.run_serial([mb])
    torch.cuda.synchronize()
    out_o, g_o = OL.layer_fwd_bwd(_oracle_cfg(cfg), w_cpu, mb_cpu, dtype=oracle_dtype, round_to=round_to)
    dt = cfg.params_dtype
    errs = {"out": assert_close(outs[0], out_o, dt, "layer out"), "dx": assert_close(dxs[0], g_o["x"], dt, "dx")}
    for k in GRAD_KEYS:
        errs[k] = assert_close(w[k].main_grad, g_o[k], dt, f"d{k}")
    print("layer rel err:", {k: f"{v:.2e}" for k, v in errs.items()})
    if round_to is not None:
        # ... and against the oracle that rounds NOWHERE: the rounding oracle above places its rounding points where
        # the pipeline stores 16-bit tensors, so a drift of the whole 16-bit pipeline would pass it.  The distance to
        # the exact result is what a chain of a dozen 16-bit stores may cost, no more.
        out_x, g_x = OL.layer_fwd_bwd(_oracle_cfg(cfg), w_cpu, mb_cpu, dtype=oracle_dtype, round_to=None)
        far = {"out": rel_err(outs[0], out_x), "dx": rel_err(dxs[0], g_x["x"])}
        far.update({k: rel_err(w[k].main_grad, g_x[k]) for k in GRAD_KEYS})
        print("layer rel err vs the unrounded oracle:", {k: f"{v:.2e}" for k, v in far.items()})
        for k, v in far.items():
            assert v <= UNROUNDED_BOUND[dt], f"{k}: {v:.3e} from the unrounded oracle > {UNROUNDED_BOUND[dt]:.1e}"


def test_layer_fp32_parity_config():
    """hidden 1024, 16 x 64 MHA, FFN 2816, b 2, s 512, fp32: rel-err <= 1e-5 on out and all grads."""
    from dhellam_amd.core.layer import small_fp32_layer
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        _check_layer(small_fp32_layer(), torch.float64)
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev


def test_layer_bf16_small_gqa_sp():
    """A scaled-down sequence-parallel GQA shard (tp 4, one kv group per rank) in bf16."""
    from dhellam_amd.core.dstb import LayerConfig
    cfg = LayerConfig(hidden_size=2048, num_attention_heads=32, num_query_groups=4, ffn_hidden_size=4096,
                      seq_length=512, micro_batch_size=1, tensor_model_parallel_size=4, tp_rank=1,
                      rope_theta=500000.0, params_dtype=torch.bfloat16)   # head_dim 64, 8 q + 1 kv per rank
    _check_layer(cfg, torch.float64, round_to=torch.bfloat16)


def test_layer_70b_shard_full_shape():
    """The headline shape: hidden 8192, 8 q + 1 kv heads x 128, FFN shard 3584, seq 4096, SP rows 512, bf16.
    Oracle in fp32 on the CPU (seconds) that stores what a bf16 pipeline stores in bf16: every op's output on
    the way forward and the gradient that comes back through it.  Output and every gradient: 1e-2."""
    from dhellam_amd.core.layer import llama70b_tp8_shard
    _check_layer(llama70b_tp8_shard(), torch.float32, round_to=torch.bfloat16)


def _ring_layer_cfg(seq, cp_rank, hidden=4096, ffn=2048):
    """A layer whose attention is the ring configuration: 32 q / 8 kv heads of 128, cp = 4, local sequence ``seq``
    (the q chunk of the rank; four KV chunks of the same length visit)."""
    from dhellam_amd.core.dstb import LayerConfig
    return LayerConfig(hidden_size=hidden, num_attention_heads=hidden // 128, num_query_groups=hidden // 512,
                       ffn_hidden_size=ffn, seq_length=seq, micro_batch_size=1, tensor_model_parallel_size=1,
                       context_parallel_size=4, cp_rank=cp_rank, rope_theta=500000.0, params_dtype=torch.bfloat16)


@pytest.mark.parametrize("cp_rank", [0, 1, 3])
def test_layer_with_ring_attention_through_the_runtime(cp_rank):
    """The ring step inside the layer, driven by the runtime's cp_attn_block_fwd_1..4 / cp_attn_block_bwd_1..5 ops
    (op ids 29 / 30), against the oracle layer whose attention is ONE dense causal attention over the zig-zag
    positions of all four chunks.  Small hidden size so that the fp64 oracle runs in seconds."""
    _check_layer(_ring_layer_cfg(512, cp_rank, hidden=1024, ffn=1024), torch.float64, round_to=torch.bfloat16)


def test_ring_layer_full_shape_serial_and_double_strand_are_bit_identical():
    """The ring configuration at its full shape (32 q / 8 kv heads x 128, local q 4096, four visiting KV chunks of
    4096) inside a layer, rank 1: the double-strand schedule (ring steps of micro-batch i+1 beside the backward
    ring calls of micro-batch i) gives the bits of the serial one."""
    from dhellam_amd.core.layer import LayerRunner, make_microbatch, make_weights
    cfg = _ring_layer_cfg(4096, 1)
    w = make_weights(cfg, 0, gen_device="cuda")
    mbs = [make_microbatch(cfg, i, gen_device="cuda") for i in range(3)]
    runner = LayerRunner(cfg, w)
    names = [str(o) for blk in runner.plan.dcblocks for o in (blk.stream1_op or []) + (blk.stream2_op or [])]
    assert "cp_attn_block_fwd_4" in names and "cp_attn_block_bwd_5" in names and "fl_attn" not in names
    outs_s, dxs_s = runner.run_serial(mbs)
    torch.cuda.synchronize()
    g_s = {k: v.clone() for k, v in runner.grads().items()}
    for _ in range(5):
        runner.zero_grads()
        outs_d, dxs_d = runner.run_double_strand(mbs)
        torch.cuda.synchronize()
        for a, b in zip(outs_s + dxs_s, outs_d + dxs_d):
            assert torch.equal(a, b)
        for k, v in runner.grads().items():
            assert torch.equal(v, g_s[k]), k


@pytest.mark.parametrize("seq", [1024, 4096])
def test_serial_and_double_strand_are_bit_identical(seq):
    """Same kernels, different stream order: outputs, input grads and accumulated weight grads must be
    identical bit for bit over 4 micro-batches.  seq 4096 is the double-strand configuration at its own size
    (four micro-batches of the full 70B shard layer)."""
    from dhellam_amd.core.layer import LayerRunner, llama70b_tp8_shard, make_microbatch, make_weights
    cfg = llama70b_tp8_shard(seq_length=seq)
    w = make_weights(cfg, 0, gen_device="cuda")
    mbs = [make_microbatch(cfg, i, gen_device="cuda") for i in range(4)]
    runner = LayerRunner(cfg, w)
    outs_s, dxs_s = runner.run_serial(mbs)
    torch.cuda.synchronize()
    g_s = {k: v.clone() for k, v in runner.grads().items()}
    runner.zero_grads()
    for _ in range(40):     # repeat: a race, or a library kernel whose summation order depends on what else runs, shows rarely
        outs_d, dxs_d = runner.run_double_strand(mbs)
        torch.cuda.synchronize()
        for a, b in zip(outs_s + dxs_s, outs_d + dxs_d):
            assert torch.equal(a, b)
        for k, v in runner.grads().items():
            assert torch.equal(v, g_s[k]), k
        runner.zero_grads()


def test_plan_with_deferred_wgrad_placeholders():
    from dhellam_amd.core.dstb import DEFAULT_PLAN
    from dhellam_amd.core.layer import LayerRunner, llama70b_tp8_shard, make_microbatch, make_weights
    import copy
    cfg = llama70b_tp8_shard(seq_length=512)
    plan = copy.deepcopy(DEFAULT_PLAN)
    # park the mlp_c wgrad and run it two blocks later, next to the attention backward
    plan["DCBlocks"][12][1] = ["gemm_dgrad_attn_l", "gemm_wgrad_attn_l", "attn_bwd", "gemm_wgrad_mlp_c_n"]
    w = make_weights(cfg, 0, gen_device="cuda")
    mbs = [make_microbatch(cfg, i, gen_device="cuda") for i in range(2)]
    ref = LayerRunner(cfg, w)
    ref.run_double_strand(mbs)
    torch.cuda.synchronize()
    g_ref = {k: v.clone() for k, v in ref.grads().items()}
    ref.zero_grads()
    alt = LayerRunner(cfg, w, plan=plan)
    assert "gemm_wgrad_mlp_c_n" in alt.plan.movable
    alt.run_double_strand(mbs)
    torch.cuda.synchronize()
    for k, v in alt.grads().items():
        assert torch.equal(v, g_ref[k]), k


def test_delay_and_emulated_collectives():
    """dh_delay / dh_host_delay keep a stream busy for at least the requested time, and a layer whose
    sequence-parallel stand-ins carry such delays computes the same bits."""
    import dataclasses
    from dhellam_amd import _lib
    from dhellam_amd.core.layer import LayerRunner, make_microbatch, make_weights
    lib, st = _lib.load(), torch.cuda.current_stream()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    _lib.check(lib.dh_delay(1000, st.cuda_stream))
    torch.cuda.synchronize()
    a.record()
    _lib.check(lib.dh_delay(2_000_000, st.cuda_stream))
    b.record()
    b.synchronize()
    assert 1.9 <= a.elapsed_time(b) <= 10.0, a.elapsed_time(b)     # at least the request; an idle GPU's timer runs slower
    with pytest.raises(RuntimeError):
        _lib.check(lib.dh_delay(-1, st.cuda_stream))
    from dhellam_amd.core.dstb import LayerConfig
    cfg = LayerConfig(hidden_size=512, num_attention_heads=8, num_query_groups=4, ffn_hidden_size=1024, seq_length=256,
                      micro_batch_size=1, tensor_model_parallel_size=4, tp_rank=1, rope_theta=10000.0,
                      params_dtype=torch.bfloat16)
    res = []
    a.record()
    _lib.check(lib.dh_host_delay(2_000_000, st.cuda_stream))      # the same in a host function of the stream
    b.record()
    b.synchronize()
    assert 1.9 <= a.elapsed_time(b) <= 50.0, a.elapsed_time(b)
    with pytest.raises(RuntimeError):
        _lib.check(lib.dh_host_delay(-1, st.cuda_stream))
    for us, engine in ((0.0, "kernel"), (40.0, "kernel"), (40.0, "host")):
        c = dataclasses.replace(cfg, comm_standin_us=us, comm_standin_engine=engine)
        w = make_weights(c, 0)
        mbs = [make_microbatch(c, i) for i in range(2)]
        outs, dxs = LayerRunner(c, w).run_double_strand(mbs)
        torch.cuda.synchronize()
        res.append((outs, dxs, [w[k].main_grad.clone() for k in GRAD_KEYS]))
    for other in res[1:]:
        for x, y in zip(res[0][0] + res[0][1] + res[0][2], other[0] + other[1] + other[2]):
            assert torch.equal(x, y)


def test_cu_partitioned_streams():
    """Streams bound to a subset of the compute units (the MI355X form of the reference's libsmctrl masks,
    csrc/operators/smctrl.cpp:135-160): the layer on masked compute streams, its stand-in collectives on
    streams that own the reserved compute units, gives the same bits as on ordinary streams; bad masks are
    refused."""
    import ctypes
    import dataclasses
    from dhellam_amd import _lib
    from dhellam_amd.common.streams import cu_mask_words, destroy_stream, partitioned_streams, stream_with_cu_mask
    from dhellam_amd.core.dstb import LayerConfig
    from dhellam_amd.core.layer import LayerRunner, make_microbatch, make_weights
    n_cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert cu_mask_words(64, 60, 4) == [0, 0xF0000000]
    with pytest.raises(ValueError):
        cu_mask_words(64, 60, 8)
    lib = _lib.load()
    out = ctypes.c_void_p()
    zero = (ctypes.c_uint32 * ((n_cus + 31) // 32))()
    with pytest.raises(RuntimeError):                                    # enables nothing
        _lib.check(lib.dh_stream_create_cu_mask(ctypes.cast(zero, ctypes.c_void_p), len(zero), ctypes.byref(out)))
    one = (ctypes.c_uint32 * 1)(1)
    if n_cus > 32:
        with pytest.raises(RuntimeError):                                # does not cover the device
            _lib.check(lib.dh_stream_create_cu_mask(ctypes.cast(one, ctypes.c_void_p), 1, ctypes.byref(out)))
    # a kernel on a stream of 8 compute units does the same work, later
    st = stream_with_cu_mask(cu_mask_words(n_cus, 0, 8))
    x = torch.randn(1 << 22, device="cuda")
    st.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(st):
        y = x * 2.0
    st.synchronize()
    assert torch.equal(y, x * 2.0)
    destroy_stream(st)

    cfg = LayerConfig(hidden_size=512, num_attention_heads=8, num_query_groups=4, ffn_hidden_size=1024, seq_length=256,
                      micro_batch_size=1, tensor_model_parallel_size=4, tp_rank=1, rope_theta=10000.0,
                      params_dtype=torch.bfloat16, comm_standin_us=30.0)
    from dhellam_amd.common import streams as S
    before = set(S._LIVE)              # masked streams other tests made and keep (math_sm_count caches them)
    with partitioned_streams(reserved_per_xcd=1) as ((c1, c2), comm):
        assert len(S._LIVE) == len(before) + 4
        _partitioned_checks(cfg, c1, c2, comm, lib)
    assert S._LIVE == before, "the partition's streams are ended with the block"


def _partitioned_checks(cfg, c1, c2, comm, lib):
    import dataclasses
    from dhellam_amd import _lib
    from dhellam_amd.core.layer import LayerRunner, make_microbatch, make_weights
    res = []
    for part in (False, True):
        c = dataclasses.replace(cfg, comm_streams=tuple(comm)) if part else cfg
        w = make_weights(c, 0)
        mbs = [make_microbatch(c, i) for i in range(3)]
        r = LayerRunner(c, w, stream1=c1, stream2=c2) if part else LayerRunner(c, w)
        outs, dxs = r.run_double_strand(mbs)
        torch.cuda.synchronize()
        res.append(outs + dxs + [w[k].main_grad.clone() for k in GRAD_KEYS])
    for a, b in zip(*res):
        assert torch.equal(a, b)
    # a stand-in on the reserved compute units starts when it is posted, whatever the compute streams run
    a_ = torch.randn(4096, 8192, device="cuda", dtype=torch.bfloat16)
    b_ = torch.randn(8192, 7168, device="cuda", dtype=torch.bfloat16)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    worst = 0.0
    for _ in range(3):
        with torch.cuda.stream(c1):
            for _ in range(6):
                a_ @ b_
        e0.record(comm[0])
        _lib.check(lib.dh_delay(50_000, comm[0].cuda_stream))
        e1.record(comm[0])
        torch.cuda.synchronize()
        worst = max(worst, e0.elapsed_time(e1) * 1e3)
    assert 45.0 <= worst <= 150.0, worst


def test_masked_streams_do_not_outlive_the_interpreter(tmp_path):
    """A process that makes masked streams and never destroys them by hand ends normally (exit status 0): the
    streams module ends them in an exit hook, before the runtime's own exit-time destructors run."""
    import subprocess
    import sys
    code = (
        "import torch\n"
        "from dhellam_amd.common.streams import partitioned_streams\n"
        "(c1, c2), comm = partitioned_streams()\n"
        "x = torch.ones(1 << 20, device='cuda')\n"
        "for st in (c1, c2, *comm):\n"
        "    st.wait_stream(torch.cuda.current_stream())\n"
        "    with torch.cuda.stream(st):\n"
        "        y = x * 2\n"
        "torch.cuda.synchronize()\n"
        "print('done', float(y[0]))\n")
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=110)
    assert "done 2.0" in res.stdout, res.stderr[-2000:]
    assert res.returncode == 0, (res.returncode, res.stderr[-2000:])


def test_fused_adjacent_ops_give_the_bits_of_the_separate_ops():
    """bda_attn + ln_mlp run as one kernel when a plan lists them next to each other (all built-in plans do);
    with ``fuse_adjacent`` off they run one after the other.  Same outputs and gradients, bit for bit."""
    import dataclasses
    from dhellam_amd.core.layer import LayerRunner, llama70b_tp8_shard, make_microbatch, make_weights
    res = []
    for fuse in (True, False):
        cfg = dataclasses.replace(llama70b_tp8_shard(seq_length=1024), fuse_adjacent=fuse)
        w = make_weights(cfg, 0, gen_device="cuda")
        mbs = [make_microbatch(cfg, i, gen_device="cuda") for i in range(2)]
        r = LayerRunner(cfg, w)
        outs, dxs = r.run_double_strand(mbs)
        torch.cuda.synchronize()
        res.append(outs + dxs + [w[k].main_grad.clone() for k in GRAD_KEYS])
    for a, b in zip(*res):
        assert torch.equal(a, b)


def test_weights_updated_around_the_version_counter_are_seen_by_the_next_step():
    """The projection weights are kept resident as W and W^T, and the data-gradient GEMMs read W^T.  An optimizer
    that writes through ``p.data`` (Megatron's do) does not move the tensor's version counter, so only an
    unconditional rebuild at the step boundary keeps W^T current: the step after such an update must give the
    gradients of the NEW weights: those of a layer that holds no resident transposes (the two take different GEMM
    kernels for the data gradients, so they agree to rounding; against stale weights they would not agree at all)."""
    import dataclasses
    from dhellam_amd.core.dstb import LayerConfig
    from dhellam_amd.core.layer import LayerRunner, make_microbatch, make_weights
    cfg = LayerConfig(hidden_size=1024, num_attention_heads=16, num_query_groups=2, ffn_hidden_size=2048,
                      seq_length=256, micro_batch_size=1, tensor_model_parallel_size=2, tp_rank=0,
                      rope_theta=500000.0, params_dtype=torch.bfloat16)
    assert cfg.resident_weight_transposes
    w = make_weights(cfg, 0)
    mbs = [make_microbatch(cfg, i) for i in range(2)]
    runner = LayerRunner(cfg, w)
    runner.run_double_strand(mbs)                                    # a first step with the initial weights
    new = make_weights(dataclasses.replace(cfg, resident_weight_transposes=False), 7)
    proj = ("column_attn_weight", "linear_attn_weight", "column_mlp_weight", "linear_mlp_weight")
    for k in proj:
        v0 = w[k]._version
        w[k].data.copy_(new[k])                                      # the optimizer's way: no version bump
        assert w[k]._version == v0
    runner.zero_grads()
    outs, dxs = runner.run_double_strand(mbs)
    ref = LayerRunner(dataclasses.replace(cfg, resident_weight_transposes=False), new)
    outs_r, dxs_r = ref.run_double_strand([make_microbatch(cfg, i) for i in range(2)])
    torch.cuda.synchronize()
    for i in range(2):
        assert torch.equal(outs[i], outs_r[i]), f"out[{i}]"
        assert_close(dxs[i], dxs_r[i].cpu(), cfg.params_dtype, f"dx[{i}] (a stale W^T would be off by ~1)")
    for k in GRAD_KEYS:
        assert_close(w[k].main_grad, new[k].main_grad.cpu(), cfg.params_dtype, k)
    # and a caller that opts out of the rebuild sees what the advice warns about: a stale W^T, silently
    for k in proj:
        w[k].data.copy_(make_weights(dataclasses.replace(cfg, resident_weight_transposes=False), 9)[k])
    _, dxs_stale = runner.run_double_strand(mbs, refresh_transposes=False)
    _, dxs_fresh = runner.run_double_strand(mbs)
    torch.cuda.synchronize()
    assert rel_err(dxs_stale[0], dxs_fresh[0]) > 0.1

"""The resident communication proxy: requests posted with stream writes and waited for with stream waits, carried
out by one resident kernel (stands where the reference has stream 3 and its communication handles,
dhellam/core/dstb.py:1142-1188).  Every kernel here ends by itself: the proxy's waits are bounded."""
import dataclasses

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_requests_are_served_in_order_and_take_the_requested_time():
    from dhellam_amd.common.comm_proxy import CommProxy
    proxy = CommProxy(2)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    x = torch.zeros(1 << 20, device="cuda")
    for us in (55.0, 20.0):
        proxy.launch(us)
        with torch.cuda.stream(s1):
            for _ in range(5):
                x.add_(1.0)
                proxy.collective(0, s1)
        with torch.cuda.stream(s2):
            for _ in range(3):
                proxy.collective(1, s2)
        proxy.stop([s1, s2])
        torch.cuda.synchronize()
        for slot, n in ((0, 5), (1, 3)):
            log = proxy.log(slot)
            assert len(log) == n
            for a, b in log:
                assert us <= b - a <= us + 5.0, (a, b)                    # carried out in the requested time
            assert all(log[i][1] <= log[i + 1][0] for i in range(n - 1))  # one after the other
    assert float(x[0]) == 10.0
    # a launch that gets no request ends on its stop alone, and the proxy can be launched again
    proxy.launch(10.0)
    proxy.stop([s1, s2])
    torch.cuda.synchronize()
    assert proxy.log(0) == []
    with pytest.raises(RuntimeError, match="running"):
        proxy.collective(0, s1)


def test_a_proxy_that_is_never_stopped_gives_up_and_releases_its_waiters():
    """Failure handling, forced from the host: a tiny limit and no stop.  The kernel ends by itself after the limit
    and the stream wait behind it is released."""
    from dhellam_amd import _lib
    from dhellam_amd.common.comm_proxy import CommProxy
    proxy = CommProxy(1)
    s = torch.cuda.Stream()
    proxy.launch(5.0, limit_ms=2.0)
    torch.cuda.synchronize()                      # the kernel has given up (nothing came for 2 ms)
    # a request posted now is not carried out by anybody; its wait is released by the count the kernel left behind
    proxy.collective(0, s)
    s.synchronize()
    proxy.stop([s])
    torch.cuda.synchronize()


def test_layer_with_proxy_standins_matches_the_plain_layer_bit_for_bit():
    """The stand-in collectives change WHEN things run, not what is computed: the double strand with proxy
    stand-ins gives the bits of the serial schedule without any, and every collective took its time."""
    from dhellam_amd.core.layer import LayerRunner, llama70b_tp8_shard, make_microbatch, make_weights
    cfg = llama70b_tp8_shard(seq_length=1024)
    w = make_weights(cfg, 0, gen_device="cuda")
    mbs = [make_microbatch(cfg, i, gen_device="cuda") for i in range(3)]
    plain = LayerRunner(cfg, w)
    outs_s, dxs_s = plain.run_serial(mbs)
    torch.cuda.synchronize()
    g_s = {k: v.clone() for k, v in plain.grads().items()}
    runner = LayerRunner(dataclasses.replace(cfg, comm_standin_us=30.0, comm_standin_engine="proxy"), w)
    for run in (runner.run_double_strand, runner.run_serial):
        runner.zero_grads()
        outs_d, dxs_d = run(mbs)
        torch.cuda.synchronize()
        for a, b in zip(outs_s + dxs_s, outs_d + dxs_d):
            assert torch.equal(a, b)
        for k, v in runner.grads().items():
            assert torch.equal(v, g_s[k]), k
        fwd, bwd = runner.proxy.log(0), runner.proxy.log(1)
        assert len(fwd) == 4 * len(mbs) and len(bwd) == 4 * len(mbs)      # 4 collectives per strand and micro-batch
        assert all(30.0 <= b - a <= 36.0 for a, b in fwd + bwd)

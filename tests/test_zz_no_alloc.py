"""The sort entry point that allocates nothing (``dh_moe_sort_static``: its histogram table is a device array
inside the library) against ``dh_moe_sort`` with a caller's workspace, through the C ABI, bit for bit, on two
calls in a row, the second with a smaller input (so what the first call left in the table must not be seen)."""
import numpy as np
import pytest
import torch

from dhellam_amd import _lib

pytestmark = pytest.mark.gpu


def _sort(lib, idx, E, static):
    n = idx.numel()
    dev = idx.device
    tpe = torch.full((E,), -7, dtype=torch.int32, device=dev)
    offs = torch.full((E + 1,), -7, dtype=torch.int32, device=dev)
    sidx = torch.full((max(n, 1),), -7, dtype=torch.int32, device=dev)
    dest = torch.full((max(n, 1),), -7, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    if static:
        _lib.check(lib.dh_moe_sort_static(idx.data_ptr(), tpe.data_ptr(), offs.data_ptr(), sidx.data_ptr(),
                                          dest.data_ptr(), n, E, st))
    else:
        ws = torch.empty(lib.dh_moe_sort_workspace_bytes(n, E), dtype=torch.uint8, device=dev)
        _lib.check(lib.dh_moe_sort(idx.data_ptr(), tpe.data_ptr(), offs.data_ptr(), sidx.data_ptr(), dest.data_ptr(),
                                   ws.data_ptr(), ws.numel(), n, E, st))
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in (tpe, offs, sidx, dest)]


def test_static_sort_matches_workspace_sort_on_two_calls_in_a_row():
    lib = _lib.load()
    assert lib.dh_moe_sort_static_max_assign() == 1 << 20
    rng = np.random.default_rng(0)
    # first a large list over many experts, then a smaller one over fewer: stale table entries of the first
    # call lie beyond and between the entries the second call uses
    for T, k, E in [(40000, 8, 64), (3001, 2, 8), (1, 1, 4)]:
        idx = torch.from_numpy(rng.integers(0, E, size=(T, k), dtype=np.int32)).cuda()
        got = _sort(lib, idx, E, static=True)
        want = _sort(lib, idx, E, static=False)
        for g, w, name in zip(got, want, ("tokens_per_expert", "expert_offsets", "sorted_idx", "dest_row")):
            assert np.array_equal(g, w), f"{name} differs at T={T} k={k} E={E}"
        assert int(got[0].sum()) == T * k


def test_static_sort_refuses_what_its_table_cannot_hold():
    lib = _lib.load()
    n = lib.dh_moe_sort_static_max_assign() + 1
    one = torch.zeros(8, dtype=torch.int32, device="cuda")
    rc = lib.dh_moe_sort_static(one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(), n, 8,
                                torch.cuda.current_stream().cuda_stream)
    assert rc == -1 and "static table" in lib.dh_last_error().decode()

"""The entry point that allocates nothing (``fsta_dfs_order_static``) against ``fsta_dfs_order``.

Through the C ABI: same parent arrays, results compared bit for bit, two calls in a row with the
second tree smaller than the first (the library's scratch array keeps the first call's contents).
Both trees are larger than what the single-workgroup kernel takes, so both calls use the scratch.
"""
import numpy as np
import pytest
import torch

from fstattention_amd import _lib, trees

pytestmark = pytest.mark.gpu


def _order(lib, entry, parent, light_first, workspace):
    n = parent.shape[0]
    perm = torch.full((n,), -7, dtype=torch.int64, device="cuda")
    rank = torch.full((n,), -7, dtype=torch.int64, device="cuda")
    status = torch.zeros((1,), dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    if entry == "static":
        rc = lib.fsta_dfs_order_static(parent.data_ptr(), n, light_first, perm.data_ptr(), rank.data_ptr(),
                                       status.data_ptr(), stream)
    else:
        rc = lib.fsta_dfs_order(parent.data_ptr(), n, light_first, perm.data_ptr(), rank.data_ptr(),
                                workspace.data_ptr(), status.data_ptr(), stream)
    _lib.check(rc)
    torch.cuda.synchronize()
    return perm.cpu().numpy(), rank.cpu().numpy(), int(status.item())


def test_static_scratch_entry_point_matches_the_workspace_one():
    lib = _lib.load()
    limit = 16384
    for n, seed, window, light in ((12000, 5, 64, 1), (5000, 6, None, 0), (limit, 7, 8, 1), (4097, 8, 200, 0), (300, 9, 16, 1)):
        host_parent = trees.random_recursive_parents(n, seed, window)
        parent = torch.from_numpy(host_parent).cuda()
        work = torch.full((_lib.dfs_order_workspace_ints(n),), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
        want = _order(lib, "workspace", parent, light, work)
        got = _order(lib, "static", parent, light, None)
        assert got[2] == 0 and want[2] == 0
        np.testing.assert_array_equal(got[0], want[0], err_msg=f"perm, n={n}")
        np.testing.assert_array_equal(got[1], want[1], err_msg=f"rank, n={n}")
        np.testing.assert_array_equal(got[0], trees.dfs_order(host_parent, "light_first" if light else "index"))
    # beyond the array's size: refused on the host, nothing launched; a malformed tree is flagged as by the other entry point
    assert lib.fsta_dfs_order_static(parent.data_ptr(), limit + 1, 0, 8, 8, 8, None) == _lib.EUNSUPPORTED
    assert b"scratch" in lib.fsta_last_error()
    bad = torch.from_numpy(trees.random_recursive_parents(6000, 3, 32)).cuda()
    bad[100] = 5000
    assert _order(lib, "static", bad, 0, None)[2] & _lib.PRE_BAD_NODE_ID


def test_status_bits_of_an_earlier_stage_do_not_change_the_order():
    """Stages of a front-end chain may share one status word: a bit another stage left there says
    nothing about this parent array, in the single-workgroup path (n <= 4096) and in the multi-launch one."""
    lib = _lib.load()
    for n in (3000, 6000):
        host_parent = trees.random_recursive_parents(n, 11, 48)
        parent = torch.from_numpy(host_parent).cuda()
        perm = torch.full((n,), -7, dtype=torch.int64, device="cuda")
        rank = torch.full((n,), -7, dtype=torch.int64, device="cuda")
        status = torch.full((1,), _lib.PRE_TOO_MANY_ANCESTORS, dtype=torch.int32, device="cuda")
        work = torch.empty((_lib.dfs_order_workspace_ints(n),), dtype=torch.int32, device="cuda")
        _lib.check(lib.fsta_dfs_order(parent.data_ptr(), n, 1, perm.data_ptr(), rank.data_ptr(), work.data_ptr(),
                                      status.data_ptr(), torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert int(status.item()) == _lib.PRE_TOO_MANY_ANCESTORS
        np.testing.assert_array_equal(perm.cpu().numpy(), trees.dfs_order(host_parent, "light_first"), err_msg=f"n={n}")


def test_static_entry_point_recorded_into_a_graph():
    """After one call outside capture (which looks the scratch array's address up), two calls -- the larger tree
    first -- are captured into one HIP graph, replayed several times with eager work in between, and compared
    with ``fsta_dfs_order`` after every replay."""
    lib = _lib.load()
    trees_ = [trees.random_recursive_parents(n, seed, 64) for n, seed in ((9000, 21), (4500, 22))]
    parents = [torch.from_numpy(t).cuda() for t in trees_]
    want = []
    for p in parents:
        work = torch.empty((_lib.dfs_order_workspace_ints(p.shape[0]),), dtype=torch.int32, device="cuda")
        want.append(_order(lib, "workspace", p, 1, work))
    _order(lib, "static", parents[1], 1, None)          # first call on this device: outside capture
    outs = [(torch.empty_like(p), torch.empty_like(p), torch.zeros((1,), dtype=torch.int32, device="cuda")) for p in parents]
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for p, (perm, rank, status) in zip(parents, outs):
                _lib.check(lib.fsta_dfs_order_static(p.data_ptr(), p.shape[0], 1, perm.data_ptr(), rank.data_ptr(),
                                                     status.data_ptr(), torch.cuda.current_stream().cuda_stream))
    for replay in range(3):
        for perm, rank, _ in outs:
            perm.fill_(-3)
            rank.fill_(-3)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for (perm, rank, status), (w_perm, w_rank, _) in zip(outs, want):
            assert int(status.item()) == 0
            np.testing.assert_array_equal(perm.cpu().numpy(), w_perm, err_msg=f"replay {replay}")
            np.testing.assert_array_equal(rank.cpu().numpy(), w_rank, err_msg=f"replay {replay}")

"""The allocation-free blocked EdgeConv backward (fgnn_edgeconv_backward_blocked_static) against
fgnn_edgeconv_backward_blocked, through the C ABI: two calls in a row on the same GPU, the second with
a smaller input (the static scratch keeps the first call's contents), gradients with dyadic values so
that the scatter sums are order independent and the comparison is exact."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(b, p, k, f, seed, cross=0):
    from ae_mlsys_gnn_amd.operators.fused_edgeconv import edgeconv_native
    from ae_mlsys_gnn_amd.operators.knn import knn_graph
    gen = torch.Generator().manual_seed(seed)
    pts = (torch.rand(b, p, 3, generator=gen) * 2 - 1).to(DEV)
    src = knn_graph(pts, k)
    n = b * p
    if cross:      # some neighbours outside their cloud: exercises the overflow list in the scratch
        pick = torch.randperm(n * k, generator=gen)[:cross].to(DEV)
        src[pick] = torch.randint(0, n, (cross,), generator=gen, dtype=torch.int32).to(DEV)
    hs, hd = torch.randn(n, f, generator=gen).to(DEV), torch.randn(n, f, generator=gen).to(DEV)
    go = (torch.round(torch.randn(n, f, generator=gen) * 8) / 8).to(DEV)
    _, arg = edgeconv_native.edgeconv_forward(k, src, hs, hd)
    return n, f, p, arg, go


def _both(n, f, block, arg, go):
    from ae_mlsys_gnn_amd import _lib
    l = _lib.lib()
    want = torch.empty(n, f, device=DEV)
    ws, wsb = _lib.workspace(l.fgnn_edgeconv_backward_blocked_workspace_bytes(n, f), go.device)
    _lib.check(l.fgnn_edgeconv_backward_blocked(n, n, f, block, _lib.ptr(arg), _lib.ptr(go), _lib.ptr(want), _lib.ptr(ws), wsb, _lib.stream_ptr()),
               "fgnn_edgeconv_backward_blocked")
    got = torch.full((n, f), float("nan"), device=DEV)
    _lib.check(l.fgnn_edgeconv_backward_blocked_static(n, n, f, block, _lib.ptr(arg), _lib.ptr(go), _lib.ptr(got), _lib.stream_ptr()),
               "fgnn_edgeconv_backward_blocked_static")
    torch.cuda.synchronize()
    return got, want


def test_static_scratch_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    from ae_mlsys_gnn_amd import _lib
    l = _lib.lib()
    # first call: 8 clouds x 1024 points, 64 features, 3000 neighbours outside their cloud (a long overflow list)
    n, f, block, arg, go = _case(8, 1024, 20, 64, seed=1, cross=3000)
    got, want = _both(n, f, block, arg, go)
    assert torch.equal(got, want)
    # second call, smaller, fewer overflow entries: nothing of the first call's list may leak in
    n2, f2, block2, arg2, go2 = _case(3, 256, 8, 24, seed=2, cross=40)
    got2, want2 = _both(n2, f2, block2, arg2, go2)
    assert torch.equal(got2, want2)
    # and without any overflow at all
    n3, f3, block3, arg3, go3 = _case(2, 128, 5, 8, seed=3)
    got3, want3 = _both(n3, f3, block3, arg3, go3)
    assert torch.equal(got3, want3)
    # the first case again: same result as before
    got4, _ = _both(n, f, block, arg, go)
    assert torch.equal(got4, want)
    # sizes beyond the static scratch are refused with a clear error, nothing is launched
    cap = l.fgnn_edgeconv_backward_blocked_static_max_elems()
    assert cap == 4 * 1024 * 1024
    big_n = cap // 64 + 1024
    rc = l.fgnn_edgeconv_backward_blocked_static(big_n, big_n, 64, 1024, _lib.ptr(arg), _lib.ptr(go), _lib.ptr(got), _lib.stream_ptr())
    assert rc == -4 and b"exceeds the static scratch" in l.fgnn_last_error()

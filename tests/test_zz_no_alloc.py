"""The allocation-free blocked EdgeConv backward (fgnn_edgeconv_backward_blocked_static) against
fgnn_edgeconv_backward_blocked, through the C ABI: two calls in a row on the same GPU, the second with
a smaller input (the static scratch keeps the first call's contents), gradients with dyadic values so
that the scatter sums are order independent and the comparison is exact.  Then the claim itself: free device
memory and torch's allocator are unchanged across the calls, and a call captured into a HIP graph (where no
allocation is possible) replays to the CPU oracle's result."""
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


def _static_call(n, f, block, arg, go, out):
    from ae_mlsys_gnn_amd import _lib
    _lib.check(_lib.lib().fgnn_edgeconv_backward_blocked_static(n, n, f, block, _lib.ptr(arg), _lib.ptr(go), _lib.ptr(out), _lib.stream_ptr()),
               "fgnn_edgeconv_backward_blocked_static")


def test_static_scratch_entry_point_allocates_nothing():
    """Free device memory (hipMemGetInfo: sees every allocation of the process, the library's own hipMalloc included) and
    torch's allocator statistics before and after a series of calls, following one warm-up call; the shapes include one that
    takes the plain fill-and-scatter form beyond the scratch size (no scratch needed, so no limit applies)."""
    from ae_mlsys_gnn_amd import _lib
    n, f, block, arg, go = _case(8, 1024, 20, 64, seed=11, cross=2000)
    n2, f2, block2, arg2, go2 = _case(3, 256, 8, 24, seed=12, cross=10)
    out, out2 = torch.empty(n, f, device=DEV), torch.empty(n2, f2, device=DEV)
    big = 70000                                   # big * 64 > 4 Mi elements; block 8192 has no LDS tile: plain form
    arg_big = torch.randint(0, big, (big, 64), dtype=torch.int32, device=DEV)
    go_big = (torch.round(torch.randn(big, 64, device=DEV) * 8) / 8)
    out_big = torch.empty(big, 64, device=DEV)
    _static_call(n, f, block, arg, go, out)       # warm-up: module load and the scratch address look-up
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    alloc0, reserved0, n_alloc0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.memory_stats()["allocation.all.allocated"]
    for _ in range(3):
        _static_call(n, f, block, arg, go, out)
        _static_call(n2, f2, block2, arg2, go2, out2)
        _static_call(big, 64, 8192, arg_big, go_big, out_big)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, "free device memory changed by %d bytes across the static calls" % (free0 - free1)
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.memory_stats()["allocation.all.allocated"]) == (alloc0, reserved0, n_alloc0)
    want = torch.zeros(big, 64, device=DEV).index_put_((arg_big.long().flatten(), torch.arange(64, device=DEV).repeat(big)), go_big.flatten(), accumulate=True)
    assert torch.equal(out_big, want)
    ws, wsb = _lib.workspace(_lib.lib().fgnn_edgeconv_backward_blocked_workspace_bytes(n, f), DEV)
    ref = torch.empty(n, f, device=DEV)
    _lib.check(_lib.lib().fgnn_edgeconv_backward_blocked(n, n, f, block, _lib.ptr(arg), _lib.ptr(go), _lib.ptr(ref), _lib.ptr(ws), wsb, _lib.stream_ptr()), "blocked")
    assert torch.equal(out, ref)


def test_static_scratch_entry_point_replays_from_a_hip_graph_to_the_oracle_result():
    """One call captured into a HIP graph after a warm-up call outside the capture; every replay (new gradients in the
    captured buffer, eager work and synchronisations between the replays) against the CPU oracle's scatter, exactly
    (dyadic gradients)."""
    from oracle import fgnn_oracle as orc
    n, f, block, arg, go = _case(4, 512, 12, 32, seed=21, cross=500)
    out = torch.full((n, f), float("nan"), device=DEV)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        _static_call(n, f, block, arg, go, out)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _static_call(n, f, block, arg, go, out)
    arg_cpu = arg.cpu()
    for rep in range(4):
        go.copy_(torch.round(torch.randn(n, f, device=DEV) * 8) / 8)
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        want = orc.edgeconv_backward(arg_cpu, go.cpu().double(), n)[0]
        assert torch.equal(out.cpu().double(), want), "replay %d differs from the oracle" % rep
        _static_call(n // 2, f, block, arg[: n // 2].contiguous() % (n // 2), go[: n // 2].contiguous(), torch.empty(n // 2, f, device=DEV))   # eager work on the same scratch
        torch.cuda.synchronize()

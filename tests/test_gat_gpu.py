"""GPU parity of the fused GAT operators against the float64 oracle (through the C ABI)."""
import pytest
import torch

from oracle import fgnn_oracle as orc
from tests.util import assert_close, assert_close_sum, c_exp, degree_edge_graph, gat_inputs, custom_graph
from ae_mlsys_gnn_amd import graphs

pytestmark = pytest.mark.gpu


def _oracle_fwd_bwd(g, x, ar, ac, go, slope):
    x = x.clone().requires_grad_(True)
    ar = ar.clone().requires_grad_(True)
    ac = ac.clone().requires_grad_(True)
    out = orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, slope, x)
    out.backward(go)
    return out.detach(), x.grad, ar.grad, ac.grad


def _check(got, ref, g, x, ar, ac, go, slope, tag=""):
    """The four results against the oracle under the derived bar: rtol 1e-4 plus the rounding scale of
    each output's own sum of absolute summands (1e-5 at least)."""
    s = orc.gat_abs_sums(ar, ac, g.row_ptr, g.col_ind, slope, x, go)
    c = c_exp(float(ar.abs().max() + ac.abs().max()))
    for val, want, name in zip(got, ref, ("out", "grad_feat", "grad_attn_row", "grad_attn_col")):
        assert_close_sum(val, want, s[name], name + tag, c=c)


def _run(g, h, f, slope=0.2, seed=0, attn_scale=1.0, variant="sm", seg_len=None, monkeypatch=None):
    from ae_mlsys_gnn_amd.operators import fused_gat as fg
    g = graphs.add_csc_torch(g)
    x, ar, ac, go = gat_inputs(g, h, f, seed, attn_scale)
    ref = _oracle_fwd_bwd(g, x, ar, ac, go, slope)
    dev = torch.device("cuda:0")
    gd = g.to(dev)
    xd = x.float().to(dev).requires_grad_(True)
    ard = ar.float().to(dev).requires_grad_(True)
    acd = ac.float().to(dev).requires_grad_(True)
    if variant == "sm":
        out = fg.fused_gat_op(ard, acd, gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, slope, xd)
    elif variant == "pipeline":
        out = fg.fused_gat_operator_pipeline(ard, acd, gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, slope, xd, gd.permute)
    elif variant == "stash":
        out = fg.fused_gat_stash_op(ard, acd, gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, slope, xd, gd.permute)
    else:
        out = fg.fused_gat_fusescatter(ard, acd, gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, slope, xd, gd.permute)
    out.backward(go.float().to(dev))
    torch.cuda.synchronize()
    _check((out, xd.grad, ard.grad, acd.grad), ref, g, x, ar, ac, go, slope)


@pytest.mark.parametrize("h,f", [(8, 32), (4, 16), (1, 64), (1, 47), (3, 20), (4, 128), (8, 128), (2, 65), (1, 1),
                                 (1, 128), (2, 16), (1, 4), (8, 4), (1, 12), (5, 24)])
def test_gat_shapes(h, f):
    g = graphs.rmat_graph(600, 12000, seed=3)
    _run(g, h, f)


@pytest.mark.parametrize("variant", ["sm", "stash", "fusescatter"])
def test_gat_variants_degree_edges(variant):
    _run(degree_edge_graph(), 8, 32, variant=variant)


@pytest.mark.parametrize("variant", ["sm", "stash", "fusescatter"])
@pytest.mark.parametrize("h,f", [(1, 128), (4, 16), (2, 8)])
def test_gat_rows_narrower_than_a_wave(h, f, variant, monkeypatch):
    """H*F <= 128: 2, 4 or 8 edges share a load instruction; degrees 0..3000, split rows and an
    XCD-aware schedule included."""
    from ae_mlsys_gnn_amd import _lib
    _run(degree_edge_graph(seed=11), h, f, variant=variant)
    monkeypatch.setenv("FGNN_SEG_LEN", "256")
    _lib.clear_schedule_cache()
    _run(degree_edge_graph(seed=12), h, f, variant=variant)
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    _lib.clear_schedule_cache()
    _run(graphs.rmat_graph(2000, 150000, seed=13), h, f, variant=variant)
    _lib.clear_schedule_cache()


def _long_row_graph(seed):
    """300 rows: the degrees of degree_edge_graph (0 ... 513 and a hub of 3000) and 280 rows of 256..300 DISTINCT sources
    (a row that names a source many times makes the rounding errors of the per-node terms add up in step, which the
    sum-of-magnitudes bar of these tests does not model)."""
    import numpy as np
    gen = np.random.default_rng(seed)
    base = degree_edge_graph(n=20, seed=seed)
    rows = []
    for i in range(20):
        d = int(base.row_ptr[i + 1] - base.row_ptr[i])
        rows.append(list(gen.choice(300, size=d, replace=False) if d <= 300 else gen.integers(0, 300, size=d)))
    rows += [list(gen.choice(300, size=int(gen.integers(256, 301)), replace=False)) for _ in range(280)]
    return custom_graph(rows, 300)


@pytest.mark.parametrize("variant", ["sm", "stash"])
@pytest.mark.parametrize("h,f", [(8, 32), (4, 64), (1, 256), (2, 72), (5, 52), (16, 32), (16, 16), (3, 50), (7, 36), (64, 16), (33, 31),
                                 (1, 128), (1, 44), (1, 64), (2, 64), (2, 24), (1, 16), (1, 32), (3, 40), (4, 16), (1, 4)])
def test_gat_long_rows_pair_layout(h, f, variant, monkeypatch):
    """Graphs averaging 64 or more entries per row take the kernels that compute the attention weights
    once per (edge, head) on one lane and hand them to the feature lanes (where edges-per-batch x heads
    fits the wave; (16, 16), (33, 31) and (4, 16) do not and keep the per-lane form), in the kernels for
    wide rows and in the packed ones for H*F <= 128.  Degrees 0..3000 with ragged batch tails, whole and
    split rows, and an XCD-aware schedule."""
    from ae_mlsys_gnn_amd import _lib
    g = _long_row_graph(seed=21)
    assert g.n_edges >= 256 * g.n          # below 256 entries per row the packed widths take the kernels of the next test
    _run(g, h, f, variant=variant)
    monkeypatch.setenv("FGNN_SEG_LEN", "256")
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    _lib.clear_schedule_cache()
    _run(_long_row_graph(seed=22), h, f, variant=variant)
    _lib.clear_schedule_cache()


@pytest.mark.parametrize("variant", ["sm", "stash"])
@pytest.mark.parametrize("h,f", [(1, 47), (1, 16), (8, 4), (2, 12), (1, 4), (1, 64), (3, 20), (2, 32), (4, 16), (1, 128), (5, 24), (4, 32), (8, 16)])
def test_gat_lane_groups_on_their_own_items(h, f, variant, monkeypatch):
    """H*F <= 128 on graphs of short rows (under 256 entries per row for 8 or 4 lane groups, under 64 for 2): every
    lane group of a wave walks a work item of its own.  Groups of 8, 16 and 32 lanes; heads of a power of two of
    lanes and of 3, 5, 6 and 12 lanes; whole rows of 0..3000 entries side by side in one wave, split rows, XCD-aware
    lists whose groups take their items from one bucket, a list shorter than one wave's groups, and a slope above 1."""
    from ae_mlsys_gnn_amd import _lib
    _lib.clear_schedule_cache()
    _run(degree_edge_graph(seed=41), h, f, variant=variant)
    _run(custom_graph([[0, 1], [], [2]], 3), h, f, variant=variant)
    _run(degree_edge_graph(seed=44), h, f, variant=variant, slope=1.5)
    monkeypatch.setenv("FGNN_SEG_LEN", "256")
    _lib.clear_schedule_cache()
    g = degree_edge_graph(n=140, seed=42)
    assert 32 * g.n <= g.n_edges < 64 * g.n
    _run(g, h, f, variant=variant)
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    _lib.clear_schedule_cache()
    _run(graphs.rmat_graph(2000, 60000, seed=43), h, f, variant=variant)
    _run(degree_edge_graph(n=150, seed=45), h, f, variant=variant)
    _lib.clear_schedule_cache()


def test_xcd_aware_schedule_is_chosen_by_row_length_skew(monkeypatch):
    """Without an override the operators take the XCD-aware work list on graphs where the rows longer
    than 64 entries hold a quarter of the entries and the longest row is 4x the mean (an R-MAT graph of
    average degree 5 qualifies, a uniform graph of average degree 100 does not); the decision is cached
    per pointer array, the results agree with the oracle either way, and FGNN_XCD_BUCKETS overrides."""
    from ae_mlsys_gnn_amd import _lib
    monkeypatch.delenv("FGNN_XCD_BUCKETS", raising=False)
    monkeypatch.delenv("FGNN_BUCKET_MIN_DEG", raising=False)
    _lib.clear_schedule_cache()
    skewed_host, flat_host = graphs.rmat_graph(20000, 100000, seed=31), graphs.uniform_graph(3000, 300000, seed=32)
    skewed, flat, short = skewed_host.to("cuda:0"), flat_host.to("cuda:0"), graphs.uniform_graph(3000, 30000, seed=33).to("cuda:0")
    assert _lib.xcd_buckets_enabled(skewed.row_ptr) is True
    assert _lib.xcd_buckets_enabled(flat.row_ptr) is False and _lib.xcd_buckets_enabled(short.row_ptr) is False
    assert len(_lib._bucket_rule_cache) == 3
    assert _lib.xcd_buckets_enabled(skewed.row_ptr) is True and len(_lib._bucket_rule_cache) == 3
    assert _lib.schedule_for(skewed.row_ptr, idx_tensor=skewed.col_ind).n_partials > 0
    assert _lib.schedule_for(flat.row_ptr, idx_tensor=flat.col_ind).n_partials == 0
    for g in (skewed_host, flat_host):
        _run(g, 4, 16, variant="sm")
        _run(g, 2, 64, variant="stash")
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "0")
    assert _lib.xcd_buckets_enabled(skewed.row_ptr) is False
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    assert _lib.xcd_buckets_enabled(flat.row_ptr) is True
    _lib.clear_schedule_cache()


def test_gat_split_rows(monkeypatch):
    monkeypatch.setenv("FGNN_SEG_LEN", "256")
    from ae_mlsys_gnn_amd import _lib
    _lib.clear_schedule_cache()
    _run(degree_edge_graph(seed=5), 8, 32)
    _run(degree_edge_graph(seed=6), 1, 47)
    _lib.clear_schedule_cache()


def test_gat_large_attention():
    # wide score range: the softmax must stay stable (no overflow, no NaN).  Scores of magnitude ~150
    # carry an fp32 rounding error of 150 * 2^-24 ~ 1e-5 before the exponential, i.e. a relative error
    # of that size in every attention weight: the bar's constant grows with max|score| (c_exp).
    _run(graphs.rmat_graph(500, 8000, seed=9), 4, 32, attn_scale=30.0)


def test_gat_self_loops_only_is_identity():
    # the 4-node graph of the reference's script/inference/gatconv_test.py:75-76
    from ae_mlsys_gnn_amd.operators import fused_gat as fg
    g = custom_graph([[0], [1], [2], [3]])
    g = graphs.add_csc_torch(g).to("cuda:0")
    x = torch.randn(4, 2, 8, device="cuda:0")
    ar = torch.randn(4, 2, device="cuda:0")
    ac = torch.randn(4, 2, device="cuda:0")
    out = fg.fused_gat_op(ar, ac, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, 0.2, x)
    assert torch.equal(out, x)


def test_gat_c1_config():
    # benchmark configuration 1: N=4096, 32k uniform edges + self loops, 4 heads x 16
    _run(graphs.uniform_graph(4096, 32768, seed=0), 4, 16)


@pytest.mark.parametrize("h,f", [(8, 32), (1, 47), (4, 128)])
def test_gat_xcd_bucketed_schedule(h, f, monkeypatch):
    # force the XCD-aware schedule on a small graph: rows above 16 entries are cut by source bucket
    from ae_mlsys_gnn_amd import _lib
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    monkeypatch.setenv("FGNN_SEG_LEN", "128")
    _lib.clear_schedule_cache()
    _run(degree_edge_graph(seed=7), h, f)
    _run(graphs.rmat_graph(3000, 200000, seed=8), h, f)
    _lib.clear_schedule_cache()


@pytest.mark.parametrize("variant", ["stash", "fusescatter"])
def test_gat_xcd_bucketed_stash_variants(variant, monkeypatch):
    # the stashed [E,H] tensors stay in the caller's edge order under a bucket-ordered schedule
    from ae_mlsys_gnn_amd import _lib
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    monkeypatch.setenv("FGNN_SEG_LEN", "128")
    _lib.clear_schedule_cache()
    _run(degree_edge_graph(seed=9), 8, 32, variant=variant)
    _run(graphs.rmat_graph(2000, 150000, seed=10), 4, 16, variant=variant)
    _lib.clear_schedule_cache()


def test_xcd_schedule_must_match_index_array():
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd._lib import lib, ptr, stream_ptr
    g = graphs.add_csc_torch(graphs.rmat_graph(500, 20000, seed=1)).to("cuda:0")
    s = _lib.Schedule(g.row_ptr, 0, g.col_ind, 16)
    other = g.col_ind.clone()
    n, h, f = g.n, 2, 8
    x = torch.randn(n, h, f, device="cuda:0"); a = torch.randn(n, h, device="cuda:0")
    out = torch.empty_like(x); m = torch.empty(n, h, device="cuda:0"); sm = torch.empty_like(m)
    ws = torch.empty(lib().fgnn_gat_forward_workspace_bytes(s.handle, h, f) // 4 + 4, device="cuda:0")
    rc = lib().fgnn_gat_forward(n, g.n_edges, h, f, ptr(a), ptr(a), ptr(g.row_ptr), ptr(other), 0.2, ptr(x), ptr(out), ptr(m),
                                ptr(sm), None, None, None, None, s.handle, ptr(ws), ws.numel() * 4, stream_ptr())
    assert rc == -6 and b"another index array" in lib().fgnn_last_error()


def test_schedule_without_positions_is_refused_by_per_edge_operators():
    """An XCD-aware schedule built without the position map serves the recomputing GAT (the default
    path of fused_gat_op) but not operators with per-edge tensors."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd._lib import lib, ptr, stream_ptr
    g = graphs.add_csc_torch(graphs.rmat_graph(500, 20000, seed=1)).to("cuda:0")
    s = _lib.Schedule(g.row_ptr, 0, g.col_ind, 16, with_positions=False)
    n, h, f = g.n, 2, 8
    x = torch.randn(n, h, f, device="cuda:0")
    att = torch.rand(g.n_edges, h, device="cuda:0")
    out = torch.empty_like(x)
    ws = torch.empty(lib().fgnn_mhspmm_workspace_bytes(s.handle, h, f) // 4 + 4, device="cuda:0")
    rc = lib().fgnn_mhspmm(n, g.n_edges, h, f, ptr(g.row_ptr), ptr(g.col_ind), None, ptr(att), ptr(x), ptr(out), s.handle, ptr(ws),
                           ws.numel() * 4, stream_ptr())
    assert rc == -6 and b"without edge positions" in lib().fgnn_last_error()
    s2 = _lib.Schedule(g.row_ptr, 0, g.col_ind, 16, with_positions=True)
    rc = lib().fgnn_mhspmm(n, g.n_edges, h, f, ptr(g.row_ptr), ptr(g.col_ind), None, ptr(att), ptr(x), ptr(out), s2.handle, ptr(ws),
                           ws.numel() * 4, stream_ptr())
    assert rc == 0


def test_gat_degenerate_graphs():
    """No edges at all, isolated nodes between connected ones, a single node with a self loop."""
    from ae_mlsys_gnn_amd.operators import fused_gat as fg
    dev = "cuda:0"
    torch.manual_seed(0)
    # (a) 5 nodes, no edges: outputs and every gradient are zero
    g = graphs.add_csc_torch(custom_graph([[], [], [], [], []])).to(dev)
    x = torch.randn(5, 2, 8, device=dev, requires_grad=True)
    a = torch.randn(5, 2, device=dev, requires_grad=True)
    b = torch.randn(5, 2, device=dev, requires_grad=True)
    out = fg.fused_gat_op(a, b, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, 0.2, x)
    out.backward(torch.ones_like(out))
    for t in (out, x.grad, a.grad, b.grad):
        assert bool(torch.isfinite(t).all()) and float(t.detach().abs().max()) == 0.0
    # (b) isolated nodes among connected ones, duplicate edges
    _run(custom_graph([[1, 1, 2], [], [0], [], [4, 0, 0, 3], []]), 2, 8)
    # (c) one node, one self loop: identity, gradients of the scores vanish
    g = graphs.add_csc_torch(custom_graph([[0]])).to(dev)
    x = torch.randn(1, 4, 16, device=dev, requires_grad=True)
    a = torch.randn(1, 4, device=dev, requires_grad=True)
    out = fg.fused_gat_op(a, a, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, 0.2, x)
    go = torch.randn_like(out)
    out.backward(go)
    # score gradients cancel up to rounding of <g, x> (magnitude ~10)
    assert torch.equal(out, x) and torch.equal(x.grad, go) and float(a.grad.abs().max()) < 1e-5


def test_gat_widest_supported_row_and_hub():
    # H*F = 1024 (the documented limit) and one destination that every node points to
    n = 3000
    rows = [[(i * 7 + 1) % n, (i * 13 + 5) % n] for i in range(n)]
    rows[17] = list(range(n))
    _run(custom_graph(rows), 8, 128)
    _run(custom_graph(rows), 16, 64)


def test_gat_negative_slope_outside_unit_interval():
    g = graphs.rmat_graph(400, 5000, seed=4)
    _run(g, 4, 16, slope=1.5)
    _run(g, 4, 16, slope=0.0)
    _run(g, 4, 16, slope=1.0)


@pytest.mark.parametrize("seed", range(12))
def test_gat_random_shapes_and_graphs(seed):
    """Seeded sweep over head counts, widths (all lane layouts: 128-bit, packed, scalar, multi-slab),
    slopes, variants and graph kinds."""
    import random
    rnd = random.Random(1000 + seed)
    h = rnd.choice([1, 1, 2, 3, 4, 5, 8, 12])
    f = rnd.choice([1, 2, 4, 7, 8, 12, 16, 20, 31, 32, 47, 64, 100, 128])
    while h * f > 1024:
        f //= 2
    slope = rnd.choice([0.2, 0.2, 0.01, 0.5, 1.0])
    variant = rnd.choice(["sm", "sm", "stash", "fusescatter"])
    kind = rnd.choice(["rmat", "uniform", "degrees"])
    if kind == "rmat":
        g = graphs.rmat_graph(rnd.randrange(50, 1500), rnd.randrange(500, 40000), seed=seed)
    elif kind == "uniform":
        g = graphs.uniform_graph(rnd.randrange(10, 3000), rnd.randrange(10, 20000), seed=seed, self_loops=rnd.random() < 0.7)
    else:
        g = degree_edge_graph(seed=100 + seed)
    _run(g, h, f, slope=slope, seed=seed, variant=variant)


@pytest.mark.parametrize("seed", range(16))
def test_gat_narrow_rows_random_graphs_and_lists(seed, monkeypatch):
    """Seeded sweep over the widths that share a wave (4 .. 128 floats per row), graph kinds (R-MAT, uniform, the degree
    ladder, short rows with a few hubs of up to 5000 entries), work-list kinds (plain or XCD-aware with several bucket
    cut-offs), segment lengths, slopes and variants: the head of a list a wave per item, the rest a lane group per item."""
    import random
    import numpy as np
    from ae_mlsys_gnn_amd import _lib
    rnd = random.Random(7000 + seed)
    if rnd.random() < 0.5:
        monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
        monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", str(rnd.choice([8, 16, 64])))
    if rnd.random() < 0.5:
        monkeypatch.setenv("FGNN_SEG_LEN", str(rnd.choice([64, 128, 256, 1024])))
    _lib.clear_schedule_cache()
    h, f = rnd.choice([(1, 4), (1, 8), (2, 4), (1, 12), (3, 4), (1, 16), (2, 8), (4, 4), (1, 20), (1, 32), (2, 16), (8, 4), (1, 44), (1, 48),
                       (3, 16), (4, 16), (1, 64), (2, 32), (3, 20), (5, 12), (1, 100), (1, 128), (2, 64), (4, 32), (8, 16), (2, 44)])
    kind = rnd.choice(["rmat", "uniform", "degrees", "hubs", "hubs"])
    if kind == "rmat":
        g = graphs.rmat_graph(rnd.randrange(50, 4000), rnd.randrange(500, 60000), seed=seed)
    elif kind == "uniform":
        g = graphs.uniform_graph(rnd.randrange(10, 3000), rnd.randrange(10, 30000), seed=seed, self_loops=rnd.random() < 0.7)
    elif kind == "degrees":
        g = degree_edge_graph(n=rnd.randrange(30, 900), seed=100 + seed)
    else:
        n = rnd.randrange(100, 2000)
        gen = np.random.default_rng(seed)
        rows = [list(gen.integers(0, n, size=int(gen.integers(0, 40)))) for _ in range(n)]
        for _ in range(rnd.randrange(1, 6)):
            rows[rnd.randrange(n)] = list(gen.integers(0, n, size=rnd.randrange(65, 5000)))
        g = custom_graph(rows, n)
    _run(g, h, f, slope=rnd.choice([0.2, 0.01, 1.0, 1.5]), seed=seed, variant=rnd.choice(["sm", "stash", "fusescatter"]))
    _lib.clear_schedule_cache()


@pytest.mark.parametrize("dense", [False, True])
@pytest.mark.parametrize("h,f", [(8, 32), (1, 128), (3, 20)])
def test_gat_without_schedules_and_reference_backward_signature(h, f, dense):
    """The C ABI as a caller with only the reference's tensors uses it: no schedules (one wave per row
    or column) and a backward that gets neither out nor the auxiliary outputs and recomputes them."""
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    g = graphs.add_csc_torch(degree_edge_graph(n=80, seed=31) if dense else graphs.rmat_graph(400, 5000, seed=31))
    x, ar, ac, go = gat_inputs(g, h, f, 3)
    ref = _oracle_fwd_bwd(g, x, ar, ac, go, 0.2)
    dev = torch.device("cuda:0")
    gd = g.to(dev)
    xd, ard, acd, god = (t.float().to(dev) for t in (x, ar, ac, go))
    out, emax, esum, _, _, _, _ = gat_native.gat_forward(ard, acd, gd.row_ptr, gd.col_ind, 0.2, xd, need_aux=False, use_schedule=False)
    gx, gar, gac = gat_native.gat_backward(0.2, gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, emax, esum, xd, ard, acd, god,
                                           use_schedule=False)
    torch.cuda.synchronize()
    _check((out, gx, gar, gac), ref, g, x, ar, ac, go, 0.2)


def test_strided_views_give_the_same_results_as_contiguous_tensors():
    """Sliced / transposed inputs (attn_row = score[:, :H], in_feat a transposed view, node_feat and pseudo
    column slices): the operators work on contiguous copies in BOTH passes, so outputs and gradients equal
    those of the contiguous tensors.  Every view's storage is at least as large as the contiguous tensor."""
    from ae_mlsys_gnn_amd.operators import fused_gat as fg
    from ae_mlsys_gnn_amd.operators import fused_gmmconv as fgm
    dev = "cuda:0"
    g = graphs.add_csc_torch(graphs.rmat_graph(300, 4000, seed=41)).to(dev)
    n, h, f = g.n, 4, 16
    torch.manual_seed(3)
    score = torch.randn(n, 2 * h, device=dev)
    xt = torch.randn(h, n, f, device=dev)
    go = torch.randn(n, h, f, device=dev)
    for variant in ("sm", "stash"):
        res = []
        for contiguous in (True, False):
            sc = score.clone().requires_grad_(True)
            xx = xt.clone().requires_grad_(True)
            ar, ac, x = sc[:, :h], sc[:, h:], xx.transpose(0, 1)
            assert not ar.is_contiguous() and not x.is_contiguous()
            if contiguous:
                ar, ac, x = ar.contiguous(), ac.contiguous(), x.contiguous()
            if variant == "sm":
                out = fg.fused_gat_op(ar, ac, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, 0.2, x)
            else:
                out = fg.fused_gat_stash_op(ar, ac, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, 0.2, x, g.permute)
            out.backward(go)
            res.append((out.detach(), sc.grad, xx.grad))
        for a, b in zip(*res):
            assert torch.equal(a, b), variant
    # the native backward with strided saved tensors (a caller of the reference's gat_backward signature)
    sc = score[:, :h]
    o = fg.gat_native.gat_forward(sc, score[:, h:], g.row_ptr, g.col_ind, 0.2, xt.transpose(0, 1))
    a = fg.gat_native.gat_backward(0.2, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o[1], o[2], xt.transpose(0, 1), sc, score[:, h:], go,
                                   out_feat=o[0], out2=o[3], cc=o[4])
    b = fg.gat_native.gat_backward(0.2, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o[1], o[2], xt.transpose(0, 1).contiguous(), sc.contiguous(),
                                   score[:, h:].contiguous(), go, out_feat=o[0], out2=o[3], cc=o[4])
    assert all(torch.equal(u, v) for u, v in zip(a, b))
    with pytest.raises(_lib_err(), match="expected"):
        fg.gat_native.gat_backward(0.2, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o[1], o[2], xt.transpose(0, 1), sc[:-1], score[:, h:], go,
                                   out_feat=o[0], out2=o[3], cc=o[4])
    # GMMConv: node_feat and pseudo as column slices of wider tensors
    k, dim = 2, 2
    wide = torch.randn(n, k, 2 * f, device=dev)
    pwide = torch.rand(g.n_edges, 2 * dim, device=dev)
    mu, isg = torch.rand(k, dim, device=dev), torch.ones(k, dim, device=dev)
    gog = torch.randn(n, k, f, device=dev)
    res = []
    for contiguous in (True, False):
        w2, p2 = wide.clone().requires_grad_(True), pwide.clone().requires_grad_(True)
        nf, ps = w2[:, :, :f], p2[:, :dim]
        if contiguous:
            nf, ps = nf.contiguous(), ps.contiguous()
        m2, s2 = mu.clone().requires_grad_(True), isg.clone().requires_grad_(True)
        out = fgm.GmmConvFuse(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute, nf, ps, m2, s2)
        out.backward(gog)
        res.append((out.detach(), w2.grad, p2.grad, m2.grad, s2.grad))
    for a, b in zip(*res):
        assert torch.equal(a, b)


def _lib_err():
    from ae_mlsys_gnn_amd._lib import FgnnError
    return FgnnError


def test_validate_graph_rejects_malformed_arrays_before_any_gather(monkeypatch):
    """fgnn_validate_graph (one reduction kernel that only reads ptr and idx themselves): a good graph passes,
    an id outside [0, n), a decreasing pointer array and a wrong end are refused with FGNN_ERR_SHAPE.  Under
    FGNN_VALIDATE=1 the operators' schedule construction runs it first, so the bad array never reaches a
    gather kernel; schedules report the device memory they hold."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.operators import fused_gat as fg
    dev = "cuda:0"
    g = graphs.add_csc_torch(graphs.rmat_graph(500, 20000, seed=42)).to(dev)
    l = _lib.lib()
    call = lambda p, i, n=g.n, e=g.n_edges: l.fgnn_validate_graph(_lib.ptr(p), _lib.ptr(i), n, n, e, _lib.stream_ptr())
    assert call(g.row_ptr, g.col_ind) == 0 and call(g.col_ptr, g.row_ind) == 0
    bad = g.col_ind.clone(); bad[123] = g.n
    assert call(g.row_ptr, bad) == -2 and b"outside" in l.fgnn_last_error()
    bad2 = g.col_ind.clone(); bad2[0] = -1
    assert call(g.row_ptr, bad2) == -2
    rp = g.row_ptr.clone(); rp[10] = rp[11] + 1
    assert call(rp, g.col_ind) == -2 and b"decreases" in l.fgnn_last_error()
    assert call(g.row_ptr, g.col_ind, e=g.n_edges - 1) == -2 and b"!= E" in l.fgnn_last_error()
    monkeypatch.setenv("FGNN_VALIDATE", "1")
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    _lib.clear_schedule_cache()
    x = torch.randn(g.n, 2, 8, device=dev)
    a = torch.randn(g.n, 2, device=dev)
    with pytest.raises(_lib.FgnnError, match="malformed graph"):
        fg.fused_gat_op(a, a, g.row_ptr, bad, g.col_ptr, g.row_ind, 0.2, x)
    out = fg.fused_gat_op(a, a, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, 0.2, x)
    assert bool(torch.isfinite(out).all())
    s = _lib.schedule_for(g.row_ptr, idx_tensor=g.col_ind, need_positions=False)
    assert s.device_bytes() >= 4 * g.n_edges + 16 * s.n_items and _lib.schedule_device_bytes() >= s.device_bytes()
    assert _lib.Schedule(g.row_ptr, 0).device_bytes() == 16 * (g.n)       # plain: one 16-byte item per row, nothing split
    _lib.clear_schedule_cache()


@pytest.mark.parametrize("h,f", [(8, 32), (1, 47), (4, 16), (3, 20)])
def test_gat_stash_in_both_orders_through_native_calls(h, f, monkeypatch):
    """The two forms of the stash behind the C ABI: the reference's (e_softmax [E,H] in CSR order from
    gat_forward, read through permute by gat_backward) and the one the autograd function keeps (in the entry
    order of the backward pass, fgnn_gat_stash_own_order, permute == NULL).  Plain, XCD-aware and no schedules;
    the own-order stash under an XCD-aware schedule is a per-column permutation of the CSC-ordered one."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    dev = torch.device("cuda:0")
    for buckets, use_schedule in (("0", True), ("1", True), ("0", False)):
        monkeypatch.setenv("FGNN_XCD_BUCKETS", buckets)
        monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
        monkeypatch.setenv("FGNN_SEG_LEN", "256")
        _lib.clear_schedule_cache()
        g = graphs.add_csc_torch(degree_edge_graph(n=300, seed=51))
        x, ar, ac, go = gat_inputs(g, h, f, 5)
        ref = _oracle_fwd_bwd(g, x, ar, ac, go, 0.2)
        alpha = orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x, return_edge=True)[2]
        gd = g.to(dev)
        xd, ard, acd, god = (t.float().to(dev) for t in (x, ar, ac, go))
        o = gat_native.gat_forward(ard, acd, gd.row_ptr, gd.col_ind, 0.2, xd, stash=True, stash_lrelu=False, use_schedule=use_schedule)
        assert_close(o[6], alpha, "e_softmax in CSR order")
        res_csr = gat_native.gat_backward(0.2, gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, o[1], o[2], xd, ard, acd, god, out_feat=o[0],
                                          out2=o[3], cc=o[4], permute=gd.permute, e_soft=o[6], use_schedule=use_schedule)
        own = gat_native.gat_stash_own_order(0.2, gd.col_ptr, gd.row_ind, o[1], o[2], ard, acd, use_schedule=use_schedule)
        res_own = gat_native.gat_backward(0.2, gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, o[1], o[2], xd, ard, acd, god, out_feat=o[0],
                                          out2=o[3], cc=o[4], e_soft=own, e_soft_order="own", use_schedule=use_schedule)
        torch.cuda.synchronize()
        for tag, res in (("CSR-ordered stash", res_csr), ("own-order stash", res_own)):
            _check((o[0],) + tuple(res), ref, g, x, ar, ac, go, 0.2, tag=" (%s, buckets %s, schedule %s)" % (tag, buckets, use_schedule))
        # the own-order stash holds alpha with the sign bit set where the pre-activation is not positive
        e_csr = orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x, return_edge=True)[1]
        csc_alpha = alpha[g.permute.long()]
        csc_signed = torch.where(e_csr[g.permute.long()] > 0, csc_alpha, -csc_alpha)
        if buckets == "0":
            assert_close(own, csc_signed, "own-order stash == signed alpha in CSC order without buckets")
        else:       # same multiset of values inside every column
            cp = g.col_ptr.long()
            seg = torch.repeat_interleave(torch.arange(g.n), cp[1:] - cp[:-1])
            a = torch.zeros(g.n, h, dtype=torch.float64).index_add_(0, seg, own.cpu().double())
            b = torch.zeros(g.n, h, dtype=torch.float64).index_add_(0, seg, csc_signed)
            assert_close(a, b, "column sums of the own-order stash")
            a = torch.zeros(g.n, h, dtype=torch.float64).index_add_(0, seg, own.cpu().double().abs())
            b = torch.zeros(g.n, h, dtype=torch.float64).index_add_(0, seg, csc_alpha)
            assert_close(a, b, "column sums of |own-order stash|")
            assert not torch.allclose(own.cpu().double(), csc_signed)
    _lib.clear_schedule_cache()


@pytest.mark.parametrize("h,f", [(8, 32), (1, 47), (4, 16)])
def test_fusescatter_pipeline_of_small_operators(h, f, monkeypatch):
    """The layer composed from the stand-alone operators (u_add_v, LeakyReLU, edge softmax, mhspmm; backward by permuted
    SpMM, SDDMM, softmax backward, row / column sums): same results as the oracle."""
    from ae_mlsys_gnn_amd import _lib
    _run(degree_edge_graph(seed=61), h, f, variant="pipeline")
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    _lib.clear_schedule_cache()
    _run(graphs.rmat_graph(1500, 90000, seed=62), h, f, variant="pipeline", slope=0.05)
    _lib.clear_schedule_cache()


@pytest.mark.parametrize("variant", ["sm", "stash"])
@pytest.mark.parametrize("h,f", [(8, 256), (4, 512), (2, 1024), (5, 300), (3, 501), (9, 128)])
def test_gat_rows_wider_than_1024_floats(h, f, variant, monkeypatch):
    """Any number of heads of up to 1024 floats each (the range of the reference's recompute and stash kernels,
    src/fused_gat/fused_gat_SM.cu:518-522): passes over groups of heads, the last group smaller than the others
    ((5, 300): 3 + 2, (3, 501): 2 + 1 in the scalar layout, (9, 128): 8 + 1), with split and merged rows and an XCD-aware
    schedule."""
    from ae_mlsys_gnn_amd import _lib
    monkeypatch.setenv("FGNN_SEG_LEN", "256")
    _lib.clear_schedule_cache()
    _run(degree_edge_graph(n=60, seed=71), h, f, variant=variant)
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    _lib.clear_schedule_cache()
    _run(graphs.rmat_graph(300, 9000, seed=72), h, f, variant=variant, slope=0.05)
    _lib.clear_schedule_cache()


def test_gat_wide_rows_through_the_reference_signatures(monkeypatch):
    """H*F > 1024 with the CSR-ordered stash of the reference's gat_forward / gat_backward pair (read through permute) and
    with a backward that is handed neither out nor the auxiliary outputs and recomputes them, group by group."""
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    h, f = 6, 256
    g = graphs.add_csc_torch(degree_edge_graph(n=50, seed=73))
    x, ar, ac, go = gat_inputs(g, h, f, 9)
    ref = _oracle_fwd_bwd(g, x, ar, ac, go, 0.2)
    gd = g.to("cuda:0")
    xd, ard, acd, god = (t.float().to("cuda:0") for t in (x, ar, ac, go))
    o = gat_native.gat_forward(ard, acd, gd.row_ptr, gd.col_ind, 0.2, xd, stash=True)
    alpha = orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x, return_edge=True)[2]
    assert_close(o[6], alpha, "e_softmax in CSR order, wide rows")
    res = gat_native.gat_backward(0.2, gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, o[1], o[2], xd, ard, acd, god, out_feat=o[0], out2=o[3],
                                  cc=o[4], permute=gd.permute, e_soft=o[6])
    _check((o[0],) + tuple(res), ref, g, x, ar, ac, go, 0.2, tag=" (wide rows, CSR-ordered stash)")
    res = gat_native.gat_backward(0.2, gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, o[1], o[2], xd, ard, acd, god)
    _check((o[0],) + tuple(res), ref, g, x, ar, ac, go, 0.2, tag=" (wide rows, recomputing backward)")


def test_gat_stash_layouts_are_not_interchangeable():
    """A CSR-ordered stash without permute is refused (by the wrapper and by the C entry) instead of being read as a stash
    in the backward pass's own order, which would take every weight from the wrong edge; the stash function writes no
    stash when nothing needs a gradient."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd._lib import check, lib, ptr, stream_ptr
    from ae_mlsys_gnn_amd.operators import fused_gat as fg
    g = graphs.add_csc_torch(graphs.rmat_graph(200, 3000, seed=74)).to("cuda:0")
    n, h, f = g.n, 4, 16
    x, ar, ac = torch.randn(n, h, f, device="cuda:0"), torch.randn(n, h, device="cuda:0"), torch.randn(n, h, device="cuda:0")
    o = fg.gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x, stash=True)
    go = torch.randn_like(x)
    with pytest.raises(_lib.FgnnError, match="needs permute"):
        fg.gat_native.gat_backward(0.2, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o[1], o[2], x, ar, ac, go, out_feat=o[0], out2=o[3], cc=o[4],
                                   e_soft=o[6])
    with pytest.raises(_lib.FgnnError, match="e_soft_order"):
        fg.gat_native.gat_backward(0.2, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o[1], o[2], x, ar, ac, go, e_soft=o[6], e_soft_order="csc")
    ws = torch.empty(lib().fgnn_gat_backward_workspace_bytes(n, h, f, None, None, 0) // 4 + 64, device="cuda:0")
    outs = [torch.empty_like(x), torch.empty_like(ar), torch.empty_like(ac)]
    rc = lib().fgnn_gat_backward(n, g.n_edges, h, f, 0.2, ptr(g.row_ptr), ptr(g.col_ind), ptr(g.col_ptr), ptr(g.row_ind), None, None, ptr(o[6]),
                                 ptr(o[1]), ptr(o[2]), ptr(x), ptr(ar), ptr(ac), ptr(o[0]), ptr(o[3]), ptr(o[4]), ptr(go), ptr(outs[0]),
                                 ptr(outs[1]), ptr(outs[2]), None, None, ptr(ws), ws.numel() * 4, stream_ptr())
    assert rc == -1 and b"fgnn_gat_backward_own_order" in lib().fgnn_last_error()
    # no gradient wanted: the stash variant keeps nothing and builds no CSC work list
    _lib.clear_schedule_cache()
    with torch.no_grad():
        out = fg.fused_gat_stash_op(ar, ac, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, 0.2, x, g.permute)
    assert torch.equal(out, o[0])
    keys = [k for k in _lib._sched_cache if k[0] == g.col_ptr.data_ptr()]
    assert not keys, "a no_grad call of the stash variant built a schedule of col_ptr"
    _lib.clear_schedule_cache()


def test_schedules_fall_back_to_plain_lists_without_the_xcd_mapping(monkeypatch):
    """fgnn_schedule_create_bucketed on a device that is not known to spread workgroups over eight XCDs (forced here with
    FGNN_XCD_MAPPING=0; the box itself reports the mapping) returns the plain list: no buckets, no index copy, and the
    operators give the same results; with the mapping the list is bucketed."""
    from ae_mlsys_gnn_amd import _lib
    g = graphs.rmat_graph(2000, 150000, seed=91)
    gd = g.to("cuda:0")
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    monkeypatch.delenv("FGNN_XCD_MAPPING", raising=False)
    _lib.clear_schedule_cache()
    s1 = _lib.Schedule(gd.row_ptr, 0, gd.col_ind, 16)
    assert s1.n_buckets == 8 and s1.device_bytes() >= 8 * g.n_edges
    prop = torch.cuda.get_device_properties(0)
    assert _lib.lib().fgnn_xcd_mapping_for(prop.gcnArchName.encode(), prop.multi_processor_count) == 8
    monkeypatch.setenv("FGNN_XCD_MAPPING", "0")
    s0 = _lib.Schedule(gd.row_ptr, 0, gd.col_ind, 16)
    assert s0.n_buckets == 0 and s0.device_bytes() < 4 * g.n_edges
    pos = s0.take_positions()
    assert torch.equal(pos, torch.arange(g.n_edges, dtype=torch.int32, device="cuda:0"))
    _lib.clear_schedule_cache()
    _run(g, 4, 16, variant="sm")
    _run(g, 2, 64, variant="stash")
    _lib.clear_schedule_cache()


def test_validation_uses_the_width_of_the_gathered_matrix(monkeypatch):
    """FGNN_VALIDATE=1 with a rectangular pattern: ids index the rows of the gathered matrix (more of them than the pointer
    array has rows: accepted; an id beyond them: refused), not the rows of the pointer array."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.operators import mhspmm as op
    monkeypatch.setenv("FGNN_VALIDATE", "1")
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    _lib.clear_schedule_cache()
    n_rows, n_cols = 50, 400
    gen = torch.Generator().manual_seed(5)
    rows = [sorted(torch.randint(0, n_cols, (30,), generator=gen).tolist()) for _ in range(n_rows)]
    g = custom_graph(rows, n_rows).to("cuda:0")
    feat = torch.randn(n_cols, 2, 8, device="cuda:0")
    out = op.mhspmm(g.row_ptr, g.col_ind, None, feat)
    ref = torch.zeros(n_rows, 16, dtype=torch.float64).index_add_(0, orc.row_of_edge(g.row_ptr.cpu()), feat.cpu().double().view(n_cols, 16)[g.col_ind.cpu().long()])
    assert_close(out.view(n_rows, 16), ref, "rectangular mhspmm under validation")
    _lib.clear_schedule_cache()
    with pytest.raises(_lib.FgnnError, match="malformed graph"):
        op.mhspmm(g.row_ptr, g.col_ind, None, feat[:300].contiguous())          # ids up to 399 against 300 rows
    _lib.clear_schedule_cache()


@pytest.mark.parametrize("n", [300, 20, 3000, 30000])
@pytest.mark.parametrize("h", [1, 3, 4, 8, 12, 20, 64])
def test_fusescatter_kernels_against_the_oracle(h, n):
    """fgnn_gat_scatter (scores + LeakyReLU + row softmax in one pass, with and without the LeakyReLU array) and
    fgnn_gat_gather_row (softmax backward + LeakyReLU backward + row sums, sign from the stashed array or formed again, out
    of place and in place) on a graph with empty rows, rows either side of the wave / workgroup threshold and a 3000-entry
    hub, against float64.  n = 20 keeps only the rows of fixed length: a mean of 430 entries per row, for which the launches
    take their dense-row configuration from 3 heads on (n = 300: only at 64 heads).  n = 3000 and 30000 add rows of 0-11
    entries until the mean row is 8 and 6 entries: short rows then share waves, 16 / 32 / 64 and 8 / 16 / 32 lanes per row
    depending on the head count."""
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    g = degree_edge_graph(n=n, seed=h)
    gen = torch.Generator().manual_seed(h)
    # scores that are exact in float32: the sign of a pre-activation (where LeakyReLU' jumps) is then the same in both precisions
    ar = torch.randn(g.n, h, generator=gen, dtype=torch.float64).float().double()
    ac = torch.randn(g.n, h, generator=gen, dtype=torch.float64).float().double()
    ge = torch.randn(g.n_edges, h, generator=gen, dtype=torch.float64)
    dst = orc.row_of_edge(g.row_ptr)
    pre = ar[dst] + ac[g.col_ind.long()]
    e_ref = torch.nn.functional.leaky_relu(pre, 0.2)
    sm_ref = orc.edge_softmax(g.row_ptr, e_ref)
    gd = g.to("cuda:0")
    ard, acd, ged = ar.float().to("cuda:0"), ac.float().to("cuda:0"), ge.float().to("cuda:0")
    el, sm = gat_native.gat_scatter(ard, acd, gd.row_ptr, gd.col_ind, 0.2, want_lrelu=True)
    _, sm2 = gat_native.gat_scatter(ard, acd, gd.row_ptr, gd.col_ind, 0.2)
    c = c_exp(float(e_ref.max() - e_ref.min()))
    one = torch.ones((), dtype=torch.float64)
    assert_close(el, e_ref, "e_lrelu of the scatter kernel")
    assert_close_sum(sm, sm_ref, one, "e_softmax of the scatter kernel", c=c)
    assert torch.equal(sm, sm2)
    # gather_row: d pre = lrelu'(pre) * sm * (ge - sum_row sm * ge)
    dot = orc.segment_sums(g.row_ptr, sm_ref * ge)
    dot_abs = orc.segment_sums(g.row_ptr, sm_ref * ge.abs())
    fac = torch.where(pre > 0, torch.ones_like(pre), torch.full_like(pre, 0.2))
    gp_ref = fac * sm_ref * (ge - dot[dst])
    gp_abs = sm_ref * (ge.abs() + dot_abs[dst])
    gar_ref, gar_abs = orc.segment_sums(g.row_ptr, gp_ref), orc.segment_sums(g.row_ptr, gp_abs)
    for elr, inplace in ((None, False), (el, False), (None, True)):
        buf = ged.clone()
        gp, gar = gat_native.gat_gather_row(0.2, gd.row_ptr, gd.col_ind, ard, acd, sm, buf, e_lrelu=elr, inplace=inplace)
        assert (gp.data_ptr() == buf.data_ptr()) == inplace
        what = " (sign %s, %s)" % ("stashed" if elr is not None else "formed again", "in place" if inplace else "out of place")
        assert_close_sum(gp, gp_ref, gp_abs, "gather_row gradient" + what, c=c)
        assert_close_sum(gar, gar_ref, gar_abs, "gather_row row sums" + what, c=c)


@pytest.mark.parametrize("h,f", [(8, 32), (1, 47), (4, 16), (3, 20)])
def test_fusescatter_variant_with_the_references_data_flow(h, f, monkeypatch):
    """FusedGATFunction: scatter kernel + mhspmm forward; permuted mhspmm, mhsddmm, gather_row and column sums backward
    (src/fused_gat/fused_gat.cu:235-326, 641-670), against the oracle, with plain and XCD-aware work lists."""
    from ae_mlsys_gnn_amd import _lib
    _run(degree_edge_graph(seed=63), h, f, variant="fusescatter")
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    monkeypatch.setenv("FGNN_SEG_LEN", "256")
    _lib.clear_schedule_cache()
    _run(graphs.rmat_graph(1500, 90000, seed=64), h, f, variant="fusescatter", slope=0.05)
    _lib.clear_schedule_cache()

"""Full-size checks at the benchmark configurations.  The 115 M-edge and 64 M-edge GAT graphs are
compared row by row and column by column with the oracle's chunked float64 restatement (run on the
device: the CPU would take minutes), for the recomputing and the stash variants; next to that,
size-independent properties of the math: attention rows sum to one, zero attention is the neighbour
mean, linearity in the features, the column-sum checksum of grad_feat, the slope == 1 shift
invariance, and the transpose round trip of csr2csc.  EdgeConv (C3, both layers of the stack) and
GMMConv (C4) are compared with the C oracle at full size."""
import time

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import fgnn_oracle as orc
from tests.util import MAX_RATIO, assert_close, assert_close_sum, c_exp
from ae_mlsys_gnn_amd import graphs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def c2_graph():
    from ae_mlsys_gnn_amd.operators import csr2csc as csc_op
    g = graphs.rmat_graph(232965, 114_600_000, seed=0, device=DEV)
    g.col_ptr, g.row_ind, g.permute = csc_op.csr2csc(g.row_ptr, g.col_ind)
    return g


def test_c2_csr2csc_properties(c2_graph):
    from ae_mlsys_gnn_amd.operators import csr2csc as csc_op
    g = c2_graph
    e = g.n_edges
    assert e == 114_600_000 + g.n
    # permute is a permutation; columns ascending; positions ascending inside a column (stable)
    pm = g.permute.long()
    assert torch.equal(torch.sort(pm).values, torch.arange(e, device=DEV))
    cols = g.col_ind.long()[pm]
    assert bool((cols[1:] >= cols[:-1]).all())
    same = cols[1:] == cols[:-1]
    assert bool((pm[1:][same] > pm[:-1][same]).all())
    assert torch.equal(g.col_ptr.long(), torch.cat([torch.zeros(1, dtype=torch.long, device=DEV),
                                                    torch.cumsum(torch.bincount(g.col_ind.long(), minlength=g.n), 0)]))
    # transpose of the transpose is the original (columns are sorted inside the rows of this graph)
    rp2, ci2, pm2 = csc_op.csr2csc(g.col_ptr, g.row_ind)
    assert torch.equal(rp2, g.row_ptr) and torch.equal(ci2, g.col_ind)
    assert torch.equal(pm[pm2.long()], torch.arange(e, device=DEV))


def test_c2_schedules_built_on_the_device_equal_the_host_built_ones(c2_graph, monkeypatch):
    """The XCD-aware work lists of the 114.8 M-edge graph (966 k items, 837 k partial segments per direction): the
    device builder and the host builder give the same items, splits and bucket-ordered index arrays."""
    from ae_mlsys_gnn_amd import _lib
    g = c2_graph
    for ptr_arr, idx in ((g.row_ptr, g.col_ind), (g.col_ptr, g.row_ind)):
        res = []
        for builder in ("device", "host"):
            monkeypatch.setenv("FGNN_SCHEDULE_BUILDER", builder)
            s = _lib.Schedule(ptr_arr, 0, idx, 0, with_positions=True)
            items, splits = s.export()
            res.append((s.n_items, s.n_partials, items, splits, s.take_positions()))
        assert res[0][:2] == res[1][:2] and res[0][1] > 100000
        assert all(torch.equal(a, b) for a, b in zip(res[0][2:], res[1][2:]))
    monkeypatch.delenv("FGNN_SCHEDULE_BUILDER")


def test_c2_gat_forward_properties(c2_graph):
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    g = c2_graph
    n, h, f = g.n, 8, 32
    torch.manual_seed(0)
    ar = torch.randn(n, h, device=DEV)
    ac = torch.randn(n, h, device=DEV)
    # (1) constant feature rows come back unchanged: attention rows sum to one
    c = torch.randn(1, h, f, device=DEV).expand(n, h, f).contiguous()
    out = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, c)[0]
    assert float((out - c).abs().max()) < 2e-5
    # (2) linearity in the features for fixed attention
    x1 = torch.randn(n, h, f, device=DEV)
    x2 = torch.randn(n, h, f, device=DEV)
    o1 = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x1)[0]
    o2 = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x2)[0]
    o12 = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x1 + 2 * x2)[0]
    assert float((o12 - (o1 + 2 * o2)).abs().max()) < 5e-5
    # (3) zero attention is the neighbour mean (reference sum built with index_add_ in edge chunks)
    z = torch.zeros(n, h, device=DEV)
    om = gat_native.gat_forward(z, z, g.row_ptr, g.col_ind, 0.2, x1)[0]
    deg = (g.row_ptr[1:] - g.row_ptr[:-1]).long()
    dst = torch.repeat_interleave(torch.arange(n, device=DEV), deg)
    acc = torch.zeros(n, h * f, dtype=torch.float64, device=DEV)
    xf = x1.view(n, h * f)
    step = 4_000_000
    for s in range(0, g.n_edges, step):
        sl = slice(s, min(s + step, g.n_edges))
        acc.index_add_(0, dst[sl], xf[g.col_ind[sl].long()].double())
    mean = (acc / deg.view(n, 1)).view(n, h, f)
    assert_close_sum(om, mean, x1.abs().max().cpu(), "neighbour mean at C2")          # scale: mean |x| <= max |x|
    # (4) stored row statistics: with zero attention max = 0 and sum = degree
    st = gat_native.gat_forward(z, z, g.row_ptr, g.col_ind, 0.2, x1)
    assert float(st[1].abs().max()) == 0.0
    assert torch.equal(st[2], deg.float().view(n, 1).expand(n, h))


def test_c2_gat_backward_properties(c2_graph):
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    g = c2_graph
    n, h, f = g.n, 8, 32
    torch.manual_seed(1)
    ar = torch.randn(n, h, device=DEV) * 0.5
    ac = torch.randn(n, h, device=DEV) * 0.5
    x = torch.randn(n, h, f, device=DEV)
    go = torch.randn(n, h, f, device=DEV)

    def run(slope, feat):
        o = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, slope, feat)
        return o, gat_native.gat_backward(slope, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o[1], o[2], feat, ar, ac, go,
                                          out_feat=o[0], out2=o[3], cc=o[4])
    # checksum: every attention row sums to one, so the column sums of grad_feat equal those of grad_out
    o, (gx, gar, gac) = run(0.2, x)
    # (scale of the checksum: sum_j sum_i alpha_ij |g_i| = sum_i |g_i|)
    assert_close_sum(gx.double().sum(0), go.double().sum(0), go.double().abs().sum(0), "sum_j grad_feat == sum_i grad_out")
    # total score gradient agrees whichever side it is summed on: sum_i grad_attn_row == sum_j grad_attn_col
    # (scale: sum over all edges of alpha |d| (geA + wsA) <= 2 sum_i max_j <|g_i|, |x_j|> <= 2 N F max|g| max|x|)
    sc = 2.0 * n * f * float(go.abs().max()) * float(x.abs().max())
    assert_close_sum(gar.double().sum(0), gac.double().sum(0), torch.tensor(sc), "sum grad_attn_row == sum grad_attn_col")
    # slope == 1: a softmax is invariant to a per-row shift, so grad_attn_row vanishes
    _, (gx1, gar1, gac1) = run(1.0, x)
    assert float(gar1.abs().max()) < 5e-4
    # grad_feat is linear in grad_out and does not depend on the features
    _, (gx2, _, _) = run(0.2, x * 3.0)
    assert torch.equal(gx2, gx)
    # constant features: out is constant, grad of the scores vanishes (every edge gives the same dot product)
    c = torch.randn(1, h, f, device=DEV).expand(n, h, f).contiguous()
    _, (_, garc, gacc) = run(0.2, c)
    assert float(garc.abs().max()) < 5e-4 and float(gacc.abs().max()) < 5e-2


def test_c2_small_operators_every_entry_vs_float64(c2_graph):
    """u_add_v, edge softmax and the multi-head SDDMM over all 114.8 M entries of the C2 graph (rows of up to 10^5
    entries: the kernels share such a row between many waves), each way, against float64 on the device."""
    from ae_mlsys_gnn_amd.operators.u_add_v import u_add_v_native
    from ae_mlsys_gnn_amd.operators.edge_softmax import edge_softmax_native
    from ae_mlsys_gnn_amd.operators import mhspmm as mh
    g = c2_graph
    n, e, h, f = g.n, g.n_edges, 8, 32
    gen = torch.Generator(device=DEV).manual_seed(5)
    ar = torch.randn(n, h, device=DEV, generator=gen)
    ac = torch.randn(n, h, device=DEV, generator=gen)
    dst = orc.row_of_edge(g.row_ptr)
    src = g.col_ind.long()
    # u_add_v forward: one fp32 addition per element, so the result is exact
    ee = u_add_v_native.u_add_v_forward(g.row_ptr, g.col_ind, ar, ac)
    assert torch.equal(ee, ar[dst] + ac[src])
    # u_add_v backward: row sums in CSR order, column sums through the transposed pattern
    ge = torch.randn(e, h, device=DEV, generator=gen)
    grow, gcol = u_add_v_native.u_add_v_backward(g.row_ptr, g.col_ind, ge)
    ged = ge.double()
    assert_close_sum(grow, orc.segment_sums(g.row_ptr, ged), orc.segment_sums(g.row_ptr, ged.abs()), "u_add_v grad row at C2", where=DEV, max_ratio=MAX_RATIO)
    gperm = ged[g.permute.long()]
    assert_close_sum(gcol, orc.segment_sums(g.col_ptr, gperm), orc.segment_sums(g.col_ptr, gperm.abs()), "u_add_v grad col at C2", where=DEV, max_ratio=MAX_RATIO)
    del gperm
    # edge softmax: exponents are differences to the row maximum, at most max - min of the inputs
    lo, hi = ee.aminmax()
    c = c_exp(float(hi - lo))
    sm = edge_softmax_native.edge_softmax(g.row_ptr, ee)
    ref, _, _ = orc._segment_softmax(ee.double(), dst, n)
    assert_close_sum(sm, ref, torch.ones((), device=DEV, dtype=torch.float64), "edge softmax at C2", c=c, where=DEV, max_ratio=MAX_RATIO)
    assert float((orc.segment_sums(g.row_ptr, sm.double()) - (g.row_ptr[1:] > g.row_ptr[:-1]).double().view(n, 1)).abs().max()) < 1e-5
    gin = edge_softmax_native.edge_softmax_backward(g.row_ptr, sm, ge)
    dot = orc.segment_sums(g.row_ptr, ref * ged)
    dot_abs = orc.segment_sums(g.row_ptr, ref * ged.abs())
    assert_close_sum(gin, ref * (ged - dot[dst]), ref * (ged.abs() + dot_abs[dst]), "edge softmax backward at C2", c=c, where=DEV, max_ratio=MAX_RATIO)
    del ref, dot, dot_abs, ged, gin, sm, ee
    # multi-head SDDMM: <a[row], b[source]> per head
    a = torch.randn(n, h, f, device=DEV, generator=gen)
    b = torch.randn(n, h, f, device=DEV, generator=gen)
    out = mh.mhsddmm(g.row_ptr, g.col_ind, a, b)
    assert_close_sum(out, orc.edge_dots(dst, src, a, b), orc.edge_dots(dst, src, a, b, absolute=True), "mhsddmm at C2", where=DEV, max_ratio=MAX_RATIO)


def test_c3_edgeconv_full_size_vs_oracle():
    from ae_mlsys_gnn_amd.operators.fused_edgeconv import edgeconv_native
    from ae_mlsys_gnn_amd.operators import knn as knn_op
    torch.manual_seed(0)
    bsz, npts, k, f = 32, 1024, 20, 64
    pts = torch.rand(bsz, npts, 3) * 2 - 1
    src = graphs.knn_graph(pts.to(DEV), k).cpu()
    theta = torch.randn(f, 3)
    phi = torch.randn(f, 3)
    x = pts.reshape(-1, 3)
    h_src = x @ theta.t()
    h_dst = x @ phi.t() - h_src
    ref_out, ref_arg = c_oracle.edgeconv_forward(k, src.numpy(), h_src.numpy(), h_dst.numpy())
    out, arg = edgeconv_native.edgeconv_forward(k, src.to(DEV), h_src.to(DEV), h_dst.to(DEV))
    assert np.array_equal(arg.cpu().numpy(), ref_arg), "argmax differs at C3"
    assert np.array_equal(out.cpu().numpy(), ref_out), "max values differ at C3"
    go = torch.randn(bsz * npts, f)
    gs = edgeconv_native.edgeconv_backward(go.to(DEV), arg, bsz * npts)
    ref_gs = c_oracle.edgeconv_backward(ref_arg, go.numpy(), bsz * npts)
    abs_gs = c_oracle.edgeconv_backward(ref_arg, go.abs().numpy(), bsz * npts)
    assert_close_sum(gs, torch.from_numpy(ref_gs), torch.from_numpy(abs_gs), "grad_src at C3", max_ratio=MAX_RATIO)
    # layer 2 of the DGCNN stack (script/train/train_edgeconv_our.py:51-56): LeakyReLU(0.2), a kNN graph rebuilt in the
    # 64-D feature space, EdgeConv(64, 64).  The graph is checked against float64 brute force, the operator
    # bit-exactly against the C oracle on the very operands the GPU used.
    h1 = torch.nn.functional.leaky_relu(out, 0.2)
    src2 = knn_op.knn_graph(h1.view(bsz, npts, f), k)
    d2 = torch.cdist(h1.view(bsz, npts, f).double(), h1.view(bsz, npts, f).double()) ** 2
    local = src2.long().view(bsz, npts, k) - (torch.arange(bsz, device=DEV) * npts).view(bsz, 1, 1)
    assert bool(((local >= 0) & (local < npts)).all())
    got_d = torch.gather(d2, 2, local)
    want_d = torch.topk(d2, k, dim=2, largest=False).values
    assert float((got_d - want_d).abs().max()) <= 1e-4 * float(want_d.max()), "feature-space kNN is not the k nearest"
    theta2 = torch.randn(f, f, device=DEV) / 8
    phi2 = torch.randn(f, f, device=DEV) / 8
    h_src2 = h1 @ theta2.t()
    h_dst2 = h1 @ phi2.t() - h_src2
    out2, arg2 = edgeconv_native.edgeconv_forward(k, src2, h_src2, h_dst2)
    ref_out2, ref_arg2 = c_oracle.edgeconv_forward(k, src2.cpu().numpy(), h_src2.cpu().numpy(), h_dst2.cpu().numpy())
    assert np.array_equal(arg2.cpu().numpy(), ref_arg2), "argmax differs at C3, layer 2"
    assert np.array_equal(out2.cpu().numpy(), ref_out2), "max values differ at C3, layer 2"
    gs2 = edgeconv_native.edgeconv_backward(go.to(DEV), arg2, bsz * npts, block=npts)
    ref_gs2 = c_oracle.edgeconv_backward(ref_arg2, go.numpy(), bsz * npts)
    abs_gs2 = c_oracle.edgeconv_backward(ref_arg2, go.abs().numpy(), bsz * npts)
    assert_close_sum(gs2, torch.from_numpy(ref_gs2), torch.from_numpy(abs_gs2), "grad_src at C3, layer 2 (blocked backward)", max_ratio=MAX_RATIO)


def test_c4_gmm_full_size_vs_oracle():
    from ae_mlsys_gnn_amd.operators import csr2csc as csc_op
    from ae_mlsys_gnn_amd.operators.fused_gmmconv import gmm_native
    n, kk, dim, f = 169343, 3, 2, 64
    g = graphs.rmat_graph(n, 2_300_000, seed=1, device=DEV)
    g.col_ptr, g.row_ind, g.permute = csc_op.csr2csc(g.row_ptr, g.col_ind)
    torch.manual_seed(2)
    deg = (g.row_ptr[1:] - g.row_ptr[:-1]).float()
    dst = torch.repeat_interleave(torch.arange(n, device=DEV), (g.row_ptr[1:] - g.row_ptr[:-1]).long())
    pseudo = torch.stack([deg[g.col_ind.long()].rsqrt(), deg[dst].rsqrt()], 1).contiguous()
    x = torch.randn(n, kk, f, device=DEV)
    mu = torch.rand(kk, dim, device=DEV)
    isg = torch.ones(kk, dim, device=DEV)
    go = torch.randn(n, kk, f, device=DEV)
    out = gmm_native.gmmconv(g.row_ptr, g.col_ind, x, pseudo, mu, isg)
    gx, gp, gm, gs = gmm_native.gmmconv_backward(g.col_ptr, g.row_ind, g.permute, x, pseudo, mu, isg, go)
    rp, ci = g.row_ptr.cpu().numpy(), g.col_ind.cpu().numpy()
    args = [t.cpu().numpy() for t in (x, pseudo, mu, isg)]
    ref = c_oracle.gmm_forward(rp, ci, *args)
    rgx, rgp, rgm, rgs = c_oracle.gmm_backward(rp, ci, *args, go.cpu().numpy())
    # bars: rtol 1e-4 plus the rounding scale of each output's sum of absolute summands (computed on the device in
    # float64 by the oracle's gmm_abs_sums); grad_mu / grad_sigma sum 2.47 M x 64 products of either sign
    sc = orc.gmm_abs_sums(g.row_ptr, g.col_ind, x.double(), pseudo.double(), mu.double(), isg.double(), go.double())
    c = c_exp(float((0.5 * (((pseudo.double().unsqueeze(1) - mu.double().unsqueeze(0)) * isg.double().unsqueeze(0)) ** 2).sum(-1)).max()))
    assert_close_sum(out, torch.from_numpy(ref), sc["out"], "gmm out at C4", c=c, max_ratio=MAX_RATIO)
    assert_close_sum(gx, torch.from_numpy(rgx), sc["grad_feat"], "gmm grad_feat at C4", c=c, max_ratio=MAX_RATIO)
    assert_close_sum(gp, torch.from_numpy(rgp), sc["grad_pseudo"], "gmm grad_pseudo at C4", c=c, max_ratio=MAX_RATIO)
    assert_close_sum(gm, torch.from_numpy(rgm), sc["grad_mu"], "gmm grad_mu at C4", c=c, max_ratio=MAX_RATIO)
    assert_close_sum(gs, torch.from_numpy(rgs), sc["grad_sigma"], "gmm grad_sigma at C4", c=c, max_ratio=MAX_RATIO)


def test_c4_graph_monet_widths_vs_oracle():
    """The C4 graph with MoNet's widths (K=2, dim=1, F=16: rows of 32 floats, eight to a load instruction): the packed SpMM
    and column pass and the passes that sum over the mixture kernels, whose short work items go a lane group each behind
    the long head of the list, against the C oracle on every row."""
    from ae_mlsys_gnn_amd.operators import csr2csc as csc_op
    from ae_mlsys_gnn_amd.operators.fused_gmmconv import gmm_native
    n, kk, dim, f = 169343, 2, 1, 16
    g = graphs.rmat_graph(n, 2_300_000, seed=1, device=DEV)
    g.col_ptr, g.row_ind, g.permute = csc_op.csr2csc(g.row_ptr, g.col_ind)
    torch.manual_seed(3)
    pseudo = torch.rand(g.n_edges, dim, device=DEV)
    x = torch.randn(n, kk, f, device=DEV)
    mu = torch.rand(kk, dim, device=DEV)
    isg = 0.5 + torch.rand(kk, dim, device=DEV)
    go = torch.randn(n, kk, f, device=DEV)
    rp, ci = g.row_ptr.cpu().numpy(), g.col_ind.cpu().numpy()
    args = [t.cpu().numpy() for t in (x, pseudo, mu, isg)]
    c = c_exp(float((0.5 * (((pseudo.double().unsqueeze(1) - mu.double().unsqueeze(0)) * isg.double().unsqueeze(0)) ** 2).sum(-1)).max()))
    for summed in (False, True):
        gout = go[:, 0, :].contiguous() if summed else go
        gfull = gout.unsqueeze(1).expand(-1, kk, -1).contiguous() if summed else go
        out = gmm_native.gmmconv(g.row_ptr, g.col_ind, x, pseudo, mu, isg, sum_kernels=summed)
        gx, gp, gm, gs = gmm_native.gmmconv_backward(g.col_ptr, g.row_ind, g.permute, x, pseudo, mu, isg, gout, sum_kernels=summed)
        ref = c_oracle.gmm_forward(rp, ci, *args)
        rgx, rgp, rgm, rgs = c_oracle.gmm_backward(rp, ci, *args, gfull.cpu().numpy())
        sc = orc.gmm_abs_sums(g.row_ptr, g.col_ind, x.double(), pseudo.double(), mu.double(), isg.double(), gfull.double())
        tag = " at the C4 graph, 2 x 16" + (" summed" if summed else "")
        ref_out, s_out = (torch.from_numpy(ref).sum(1), sc["out"].sum(1)) if summed else (torch.from_numpy(ref), sc["out"])
        assert_close_sum(out, ref_out, s_out, "gmm out" + tag, c=c, max_ratio=MAX_RATIO)
        assert_close_sum(gx, torch.from_numpy(rgx), sc["grad_feat"], "gmm grad_feat" + tag, c=c, max_ratio=MAX_RATIO)
        assert_close_sum(gp, torch.from_numpy(rgp), sc["grad_pseudo"], "gmm grad_pseudo" + tag, c=c, max_ratio=MAX_RATIO)
        assert_close_sum(gm, torch.from_numpy(rgm), sc["grad_mu"], "gmm grad_mu" + tag, c=c, max_ratio=MAX_RATIO)
        assert_close_sum(gs, torch.from_numpy(rgs), sc["grad_sigma"], "gmm grad_sigma" + tag, c=c, max_ratio=MAX_RATIO)


@pytest.fixture(scope="module")
def c5_graph():
    from ae_mlsys_gnn_amd.operators import csr2csc as csc_op
    g = graphs.rmat_graph(2449029, 61_900_000, seed=0, device=DEV)
    g.col_ptr, g.row_ind, g.permute = csc_op.csr2csc(g.row_ptr, g.col_ind)
    return g


@pytest.mark.parametrize("h,f", [(1, 47), (1, 48), (8, 32)])
def test_c5_gat_properties(c5_graph, h, f):
    """Config C5 (2,449,029 nodes, 61.9 M edges + self loops; features larger than every cache):
    layer 2 in its scalar layout (1 x 47), in the zero-padded packed layout the GAT layer uses
    (1 x 48) and layer 1 (8 x 32).  Same size-independent properties as at C2."""
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    g = c5_graph
    n = g.n
    torch.manual_seed(h * 100 + f)
    ar = torch.randn(n, h, device=DEV) * 0.5
    ac = torch.randn(n, h, device=DEV) * 0.5
    x = torch.randn(n, h, f, device=DEV)
    go = torch.randn(n, h, f, device=DEV)
    # forward: constant rows come back unchanged; zero attention is the neighbour mean
    c = torch.randn(1, h, f, device=DEV).expand(n, h, f).contiguous()
    assert float((gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, c)[0] - c).abs().max()) < 2e-5
    z = torch.zeros(n, h, device=DEV)
    om = gat_native.gat_forward(z, z, g.row_ptr, g.col_ind, 0.2, x)
    deg = (g.row_ptr[1:] - g.row_ptr[:-1]).long()
    dst = torch.repeat_interleave(torch.arange(n, device=DEV), deg)
    acc = torch.zeros(n, h * f, dtype=torch.float64, device=DEV)
    xf = x.view(n, h * f)
    for s in range(0, g.n_edges, 4_000_000):
        sl = slice(s, min(s + 4_000_000, g.n_edges))
        acc.index_add_(0, dst[sl], xf[g.col_ind[sl].long()].double())
    assert_close_sum(om[0], (acc / deg.view(n, 1)).view(n, h, f), x.abs().max().cpu(), "neighbour mean at C5")
    assert torch.equal(om[2], deg.float().view(n, 1).expand(n, h))
    del acc, dst
    # backward: column-sum checksum, both sides of the score gradient, independence of the features
    o = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x)
    gx, gar, gac = gat_native.gat_backward(0.2, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o[1], o[2], x, ar, ac, go,
                                           out_feat=o[0], out2=o[3], cc=o[4])
    assert_close_sum(gx.double().sum(0), go.double().sum(0), go.double().abs().sum(0), "sum_j grad_feat == sum_i grad_out")
    sc = 2.0 * n * f * float(go.abs().max()) * float(x.abs().max())
    assert_close_sum(gar.double().sum(0), gac.double().sum(0), torch.tensor(sc), "sum grad_attn_row == sum grad_attn_col")
    o3 = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x * 3.0)
    gx3 = gat_native.gat_backward(0.2, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o3[1], o3[2], x * 3.0, ar, ac, go,
                                  out_feat=o3[0], out2=o3[3], cc=o3[4])[0]
    assert torch.equal(gx3, gx)


def _gat_full_size_vs_float64(g, h, f, slope, seed, variants, chunk=1 << 20):
    """Every row and every column of the full-size graph against the float64 restatement
    (oracle.gat_reference_chunked, run on the device in float64): out, grad_feat, grad_attn_row and
    grad_attn_col of ALL nodes, so the hub rows and columns (split into segments, merged by the merge kernels)
    and the short ones are all covered.  Bar: rtol 1e-4 plus the rounding scale of each output's own sum of
    absolute summands."""
    from ae_mlsys_gnn_amd.operators import fused_gat as fg
    n = g.n
    gen = torch.Generator(device=DEV).manual_seed(seed)
    ar = torch.randn(n, h, device=DEV, generator=gen)
    ac = torch.randn(n, h, device=DEV, generator=gen)
    x = torch.randn(n, h, f, device=DEV, generator=gen)
    go = torch.randn(n, h, f, device=DEV, generator=gen)
    t0 = time.time()

    def log(msg):          # a line per phase: the float64 restatement of 10^8 edges takes a minute or two
        torch.cuda.synchronize()
        print("[float64 reference %dx%d, E=%d] %s at %.1f s" % (h, f, g.n_edges, msg, time.time() - t0), flush=True)
    ref = orc.gat_reference_chunked(ar, ac, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute, slope, x, go, chunk=chunk, log=log)
    log("all done")
    jumps = int((ref["A_grad_attn_row"] != 0).sum())
    print("(node, head) pairs with a pre-activation within fp32 rounding of zero: %d" % jumps, flush=True)
    ref = {k: v.cpu() for k, v in ref.items()}
    torch.cuda.empty_cache()
    c = c_exp(float(ar.abs().max() + ac.abs().max()))
    deg = (g.row_ptr[1:] - g.row_ptr[:-1])
    cdeg = (g.col_ptr[1:] - g.col_ptr[:-1])
    where = "N=%d E=%d %dx%d, longest row %d, longest column %d" % (n, g.n_edges, h, f, int(deg.max()), int(cdeg.max()))
    for variant in variants:
        xd, ard, acd = (t.clone().requires_grad_(True) for t in (x, ar, ac))
        if variant == "sm":
            out = fg.fused_gat_op(ard, acd, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, slope, xd)
        else:
            out = fg.fused_gat_stash_op(ard, acd, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, slope, xd, g.permute)
        out.backward(go)
        torch.cuda.synchronize()
        for val, name in ((out, "out"), (xd.grad, "grad_feat"), (ard.grad, "grad_attn_row"), (acd.grad, "grad_attn_col")):
            assert_close_sum(val, ref[name], ref["S_" + name], "%s [%s] at %s" % (name, variant, where), c=c, extra=ref.get("A_" + name),
                             max_ratio=MAX_RATIO)
        del out, xd, ard, acd
        torch.cuda.empty_cache()


def test_c2_gat_every_row_and_column_vs_float64(c2_graph):
    """Config C2 (232,965 nodes, 114.8 M edges, 8 x 32): recompute and stash variants."""
    _gat_full_size_vs_float64(c2_graph, 8, 32, 0.2, 7, ("sm", "stash"))


@pytest.mark.parametrize("h,f,variants", [(8, 32, ("sm", "stash")), (1, 48, ("sm",)), (1, 47, ("sm",))])
def test_c5_gat_every_row_and_column_vs_float64(c5_graph, h, f, variants):
    """Config C5 (2,449,029 nodes, 64.3 M edges): layer 1 (8 x 32), layer 2 in the zero-padded layout the GAT layer
    uses (1 x 48) and in its scalar layout (1 x 47)."""
    _gat_full_size_vs_float64(c5_graph, h, f, 0.2, 100 * h + f, variants)


def test_c2_graph_gmm_layer_two_dataflows_agree(c2_graph, monkeypatch):
    """MoNet's second layer at the reddit shape (16 -> 41, K=2, dim=1, 114.8 M edges): the layer that aggregates
    its input before the fc and the layer that transforms first (the reference's order) are the same sums in
    another order, computed by different kernels (shared-feature forward / column pass against the packed
    SpMM / summed column pass); outputs and every gradient must agree.  With the per-edge coordinates in
    the schedules' own orders on the aggregate-first side, in CSR / CSC order on the other."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.layers import GMMConv
    from ae_mlsys_gnn_amd.operators.fused_gmmconv import gmm_edge_positions
    g = c2_graph
    torch.manual_seed(7)
    layer = GMMConv(16, 41, dim=1, n_kernels=2).to(DEV)
    with torch.no_grad():
        layer.mu.uniform_(0.2, 0.8)
        layer.bias.normal_()
    feat = torch.randn(g.n, 16, device=DEV)
    pseudo = torch.rand(g.n_edges, 1, device=DEV)
    go = torch.randn(g.n, 41, device=DEV) / 16
    results = []
    for aggregate in (True, False):
        monkeypatch.setattr(GMMConv, "_aggregate_first", lambda self, x, a=aggregate: a)
        for p_ in layer.parameters():
            p_.grad = None
        fd = feat.clone().requires_grad_(True)
        if aggregate:
            pos_r, pos_c = gmm_edge_positions(g.row_ptr, g.col_ind), gmm_edge_positions(g.col_ptr, g.row_ind, summed_backward=True)
            assert pos_r is not None and pos_c is not None
            to_csc = g.permute.long()[pos_c.long()]
            pc = pseudo[to_csc].contiguous().requires_grad_(True)
            out = layer(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute, fd, pseudo[pos_r.long()].contiguous(), pseudo_csc=pc, own_order=True)
            del pos_r, pos_c
        else:
            to_csc = g.permute.long()
            pc = pseudo[to_csc].contiguous().requires_grad_(True)
            out = layer(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute, fd, pseudo, pseudo_csc=pc)
        out.backward(go)
        gp = torch.zeros(g.n_edges, 1, device=DEV)
        gp[to_csc] = pc.grad                                    # back to CSR order
        results.append([out.detach(), fd.grad, gp, layer.fc.weight.grad.clone(), layer.mu.grad.clone(), layer.inv_sigma.grad.clone(),
                        layer.bias.grad.clone()])
        del pc, to_csc, out, fd
    a, b = results
    names = ("out", "grad feat", "grad pseudo", "grad fc.weight", "grad mu", "grad inv_sigma", "grad bias")
    # Two fp32 evaluations of the same sums in different orders: each is within the derived bar of the exact value, so
    # they agree within twice that bar.  The scales (sums of absolute summands) are bounded from above with row /
    # column lengths and maxima instead of being formed per edge ([E,K,F] in float64 would be 75 GB per temporary).
    with torch.no_grad():
        kk, fo = 2, 41
        wfc, af, ag = layer.fc.weight.double().abs(), feat.double().abs(), go.double().abs()
        deg = (g.row_ptr[1:] - g.row_ptr[:-1]).double().view(-1, 1)
        cdeg = (g.col_ptr[1:] - g.col_ptr[:-1]).double().view(-1, 1)
        s_h = (af @ wfc.t()).view(g.n, kk, fo)                          # scale of the projected features
        m_h = s_h.sum(1).max(0).values                                  # [out]: max over nodes of sum_k S_h
        g_max = ag.max(0).values                                        # [out]
        t_max = 1.0                                                     # |pseudo - mu| <= 1 (both in [0, 1])
        s2 = float((layer.inv_sigma.double() ** 2).max())
        edge_gw = float((g_max * s_h.view(g.n, kk, fo).max(0).values.max(0).values).sum())   # bound of sum_o |g_o| S_h per (edge, kernel)
        w_in = wfc.view(kk, fo, -1)                                      # [K, out, in]
        scales = (deg * m_h.view(1, -1) + layer.bias.double().abs().view(1, -1),
                  cdeg * (g_max.view(1, fo, 1) * w_in).sum((0, 1)).view(1, -1),
                  torch.tensor(kk * edge_gw * t_max * s2),
                  (g_max.view(1, fo, 1) * (cdeg * af).sum(0).view(1, 1, -1)).expand(kk, fo, -1).reshape(kk * fo, -1),
                  torch.tensor(g.n_edges * edge_gw * t_max * s2), torch.tensor(g.n_edges * edge_gw * t_max * t_max * float(layer.inv_sigma.abs().max())),
                  ag.sum(0))
    c = 2 * c_exp(0.5 * s2)
    for name, x, y, sc in zip(names, a, b, scales):
        assert_close_sum(x, y, sc.cpu(), "aggregate first vs transform first: " + name, c=c)
    _lib.clear_schedule_cache()

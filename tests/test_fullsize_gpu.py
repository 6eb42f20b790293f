"""Full-size checks at the benchmark configurations.  Where the CPU oracle is too slow (the
115 M-edge GAT graph) the checks are size-independent properties of the math: attention rows sum
to one, zero attention is the neighbour mean, linearity in the features, the column-sum checksum
of grad_feat, the slope == 1 shift invariance, and the transpose round trip of csr2csc; on top of
that a sample of rows and columns of the full-size graph is compared with float64 torch math.  EdgeConv
(C3) and GMMConv (C4) are small enough to compare with the oracle at full size."""
import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import fgnn_oracle as orc
from tests.util import assert_close
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
    assert_close(om, mean, "neighbour mean at C2", atol=2e-5)
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
    assert_close(gx.double().sum(0), go.double().sum(0), "sum_j grad_feat == sum_i grad_out", rtol=1e-5, atol=1e-2)
    # total score gradient agrees whichever side it is summed on: sum_i grad_attn_row == sum_j grad_attn_col
    assert_close(gar.double().sum(0), gac.double().sum(0), "sum grad_attn_row == sum grad_attn_col", rtol=1e-4, atol=5e-2)
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


def test_c3_edgeconv_full_size_vs_oracle():
    from ae_mlsys_gnn_amd.operators.fused_edgeconv import edgeconv_native
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
    assert_close(gs, torch.from_numpy(ref_gs), "grad_src at C3", atol=1e-4)


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
    assert_close(out, torch.from_numpy(ref), "gmm out at C4", atol=1e-4)
    assert_close(gx, torch.from_numpy(rgx), "gmm grad_feat at C4", atol=1e-4)
    assert_close(gp, torch.from_numpy(rgp), "gmm grad_pseudo at C4", atol=1e-3)
    # sums over 2.47 M edges of terms of either sign
    assert_close(gm, torch.from_numpy(rgm), "gmm grad_mu at C4", rtol=1e-3, atol=1.0)
    assert_close(gs, torch.from_numpy(rgs), "gmm grad_sigma at C4", rtol=1e-3, atol=1.0)


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
    assert_close(om[0], (acc / deg.view(n, 1)).view(n, h, f), "neighbour mean at C5", atol=2e-5)
    assert torch.equal(om[2], deg.float().view(n, 1).expand(n, h))
    del acc, dst
    # backward: column-sum checksum, both sides of the score gradient, independence of the features
    o = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x)
    gx, gar, gac = gat_native.gat_backward(0.2, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o[1], o[2], x, ar, ac, go,
                                           out_feat=o[0], out2=o[3], cc=o[4])
    assert_close(gx.double().sum(0), go.double().sum(0), "sum_j grad_feat == sum_i grad_out", rtol=1e-5, atol=2e-2)
    assert_close(gar.double().sum(0), gac.double().sum(0), "sum grad_attn_row == sum grad_attn_col", rtol=1e-4, atol=5e-2)
    o3 = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x * 3.0)
    gx3 = gat_native.gat_backward(0.2, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o3[1], o3[2], x * 3.0, ar, ac, go,
                                  out_feat=o3[0], out2=o3[3], cc=o3[4])[0]
    assert torch.equal(gx3, gx)


def _segment_sums(vals, deg):
    """Sums of consecutive segments of `vals` ([P, H], float64) with lengths `deg` (all >= 1), by
    differences of a running sum (float64 index_add_ serialises on its atomics)."""
    c = torch.cumsum(vals, 0)[torch.cumsum(deg, 0) - 1]
    return c - torch.cat([torch.zeros_like(c[:1]), c[:-1]])


def _rows_float64(g, rows, ar, ac, x, slope, go=None, need_out=True):
    """Float64 restatement of the GAT math for the given destination rows only (all their edges), on
    the device with plain torch ops: returns out[rows] and, with go, grad_attn_row[rows] and the
    per-edge (position, g) pairs needed for column sums."""
    rp = g.row_ptr.long()
    deg = rp[rows + 1] - rp[rows]
    seg = torch.repeat_interleave(torch.arange(rows.numel(), device=DEV), deg)            # edge -> index into rows
    first = torch.cumsum(deg, 0) - deg                                                      # index of each row's first edge in the list
    pos = rp[rows][seg] + (torch.arange(seg.numel(), device=DEV) - first[seg])              # CSR positions of the listed edges
    src = g.col_ind[pos].long()
    e = torch.nn.functional.leaky_relu(ar[rows].double()[seg] + ac[src].double(), slope)   # [P, H]
    m = torch.full((rows.numel(), e.shape[1]), -float("inf"), dtype=torch.float64, device=DEV).scatter_reduce(
        0, seg.view(-1, 1).expand_as(e), e, "amax")
    w = torch.exp(e - m[seg])
    s = _segment_sums(w, deg)
    alpha = w / s[seg]
    h, f = x.shape[1], x.shape[2]
    out = torch.zeros(rows.numel(), h, f, dtype=torch.float64, device=DEV)
    ge = torch.empty_like(alpha) if go is not None else None
    for a in range(0, pos.numel(), 1 << 20):                                               # chunks: [P, H, F] in float64 is large
        sl = slice(a, min(a + (1 << 20), pos.numel()))
        xs = x[src[sl]].double()
        if need_out:
            out.index_add_(0, seg[sl], alpha[sl].unsqueeze(-1) * xs)
        if go is not None:
            ge[sl] = (go[rows].double()[seg[sl]] * xs).sum(-1)
    if go is None:
        return out
    ws = _segment_sums(alpha * ge, deg)
    gscore = alpha * (ge - ws[seg]) * torch.where(e > 0, 1.0, slope)
    gar = _segment_sums(gscore, deg)
    return out, gar, pos, src, seg, alpha, gscore


def test_c2_gat_sampled_rows_and_columns_vs_float64(c2_graph):
    """Direct parity at full size on a sample: 100 destination rows (forward, grad_attn_row) and 6
    source columns with all the rows they touch (grad_feat, grad_attn_col), against float64 torch math."""
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    g = c2_graph
    n, h, f, slope = g.n, 8, 32, 0.2
    gen = torch.Generator(device=DEV).manual_seed(7)
    ar = torch.randn(n, h, device=DEV, generator=gen)
    ac = torch.randn(n, h, device=DEV, generator=gen)
    x = torch.randn(n, h, f, device=DEV, generator=gen)
    go = torch.randn(n, h, f, device=DEV, generator=gen)
    o = gat_native.gat_forward(ar, ac, g.row_ptr, g.col_ind, slope, x)
    gx, gar, gac = gat_native.gat_backward(slope, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, o[1], o[2], x, ar, ac, go,
                                           out_feat=o[0], out2=o[3], cc=o[4])
    rows = torch.randperm(n, device=DEV, generator=gen)[:100]
    ref_out, ref_gar = _rows_float64(g, rows, ar, ac, x, slope, go)[:2]
    assert_close(o[0][rows], ref_out, "out on sampled rows at C2")
    scale = float(go.abs().max() * x.abs().max() * f)
    assert_close(gar[rows], ref_gar, "grad_attn_row on sampled rows at C2", atol=1e-5 * scale)
    # columns of modest length, so that the rows they touch stay a few million edges
    cp = g.col_ptr.long()
    cdeg = cp[1:] - cp[:-1]
    cand = torch.nonzero((cdeg >= 20) & (cdeg <= 60)).squeeze(1)
    cols = cand[torch.randperm(cand.numel(), device=DEV, generator=gen)[:6]]
    touched = torch.unique(torch.cat([g.row_ind[a:b].long() for a, b in zip(cp[cols].tolist(), cp[cols + 1].tolist())]))
    _, _, pos, src, seg, alpha, gscore = _rows_float64(g, touched, ar, ac, x, slope, go, need_out=False)
    for j in cols.tolist():
        mine = src == j
        rws = touched[seg[mine]]
        want_gx = (alpha[mine].unsqueeze(-1) * go[rws].double()).sum(0)
        assert_close(gx[j], want_gx, "grad_feat of column %d at C2" % j)
        assert_close(gac[j], gscore[mine].sum(0), "grad_attn_col of column %d at C2" % j, atol=1e-5 * scale)


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
    # rows sum ~490 terms of either sign; the parameter gradients sum over all nodes / all 114.8 M edges
    # (observed: 7e-4 on outputs up to 1100, 7e-5 on grad feat, 5e-7 on grad pseudo, 1.5e-3 / 3e-4 / 6e-5 on parameter
    # gradients of magnitude 500-2000)
    bars = ((1e-4, 2e-3), (1e-4, 5e-4), (1e-4, 1e-5), (1e-5, 1e-2), (1e-5, 5e-3), (1e-5, 2e-3), (1e-5, 1e-3))
    for name, x, y, (rtol, atol) in zip(names, a, b, bars):
        assert_close(x, y, "aggregate first vs transform first: " + name, rtol=rtol, atol=atol)
    _lib.clear_schedule_cache()

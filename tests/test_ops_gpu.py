"""GPU parity of EdgeConv, GMMConv, csr2csc and the small operators against the oracle,
called through the C ABI (ctypes binding of libfgnn_hip.so)."""
import numpy as np
import pytest
import torch

from oracle import fgnn_oracle as orc
from oracle import c_oracle
from tests.util import assert_close, assert_close_sum, c_exp, custom_graph, degree_edge_graph
from ae_mlsys_gnn_amd import graphs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ------------------------------------------------------------------ csr2csc (bit-exact)
@pytest.mark.parametrize("n,e,seed", [(1, 1, 0), (7, 20, 1), (300, 5000, 2), (5000, 200000, 3), (70000, 300000, 4)])
def test_csr2csc_bit_exact(n, e, seed):
    from ae_mlsys_gnn_amd.operators import csr2csc as op
    g = graphs.rmat_graph(n, e, seed=seed)
    cp, ri, pm = orc.csr2csc(g.row_ptr.numpy(), g.col_ind.numpy())
    gd = g.to(DEV)
    col_ptr, row_ind, permute = op.csr2csc(gd.row_ptr, gd.col_ind)
    assert np.array_equal(col_ptr.cpu().numpy(), cp)
    assert np.array_equal(permute.cpu().numpy(), pm)
    assert np.array_equal(row_ind.cpu().numpy(), ri)


def test_csr2csc_duplicates_unsorted_and_empty():
    from ae_mlsys_gnn_amd.operators import csr2csc as op
    # duplicate (i,j) entries, columns not sorted inside a row, empty rows and empty columns
    g = custom_graph([[3, 1, 3, 3], [], [0, 0], [4, 1], [], [1]], n=6)
    cp, ri, pm = orc.csr2csc_bruteforce(g.row_ptr.numpy(), g.col_ind.numpy())
    gd = g.to(DEV)
    col_ptr, row_ind, permute = op.csr2csc(gd.row_ptr, gd.col_ind)
    assert np.array_equal(col_ptr.cpu().numpy(), cp)
    assert np.array_equal(permute.cpu().numpy(), pm)
    assert np.array_equal(row_ind.cpu().numpy(), ri)
    # no edges at all
    g0 = custom_graph([[], [], []]).to(DEV)
    col_ptr, row_ind, permute = op.csr2csc(g0.row_ptr, g0.col_ind)
    assert col_ptr.tolist() == [0, 0, 0, 0] and row_ind.numel() == 0
    # sparsetrans carries values along
    vals = torch.arange(g.n_edges, dtype=torch.float32, device=DEV) * 0.5
    out = op.sparsetrans(gd.row_ptr, gd.col_ind, vals)
    assert torch.equal(out.cpu(), torch.from_numpy(pm).float() * 0.5)


def test_csr2csc_round_trip_large():
    # transpose of the transpose is the original (columns sorted inside rows): size-independent property
    from ae_mlsys_gnn_amd.operators import csr2csc as op
    g = graphs.rmat_graph(100000, 3000000, seed=11, device=DEV)
    col_ptr, row_ind, permute = op.csr2csc(g.row_ptr, g.col_ind)
    rp2, ci2, pm2 = op.csr2csc(col_ptr, row_ind)
    assert torch.equal(rp2, g.row_ptr) and torch.equal(ci2, g.col_ind)
    assert torch.equal(permute.long()[pm2.long()], torch.arange(g.n_edges, device=DEV))
    assert torch.equal(torch.sort(permute).values.long(), torch.arange(g.n_edges, device=DEV))


# ------------------------------------------------------------------ EdgeConv (argmax bit-exact)
def _edgeconv_case(bsz, npts, k, fin, fout, seed, quantize=False):
    gen = torch.Generator().manual_seed(seed)
    pts = torch.rand(bsz, npts, 3, generator=gen) * 2 - 1
    src = graphs.knn_graph(pts, k)
    n = bsz * npts
    h_src = torch.randn(n, fout, generator=gen)
    h_dst = torch.randn(n, fout, generator=gen)
    if quantize:   # many exact ties
        h_src = torch.round(h_src * 2) / 2
        h_dst = torch.round(h_dst * 2) / 2
    return src, h_src, h_dst


@pytest.mark.parametrize("bsz,npts,k,f,quant", [(2, 64, 5, 64, False), (3, 100, 20, 64, False), (2, 64, 7, 3, False),
                                                (2, 128, 20, 64, True), (1, 50, 33, 130, True), (1, 40, 1, 8, False)])
def test_edgeconv_forward_bit_exact(bsz, npts, k, f, quant):
    from ae_mlsys_gnn_amd.operators.fused_edgeconv import edgeconv_native
    src, h_src, h_dst = _edgeconv_case(bsz, npts, k, 3, f, seed=k + f, quantize=quant)
    ref_out, ref_arg = orc.edgeconv_forward(k, src, h_src, h_dst)
    c_out, c_arg = c_oracle.edgeconv_forward(k, src.numpy(), h_src.numpy(), h_dst.numpy())
    assert np.array_equal(ref_arg.numpy(), c_arg) and np.array_equal(ref_out.numpy(), c_out)
    out, arg = edgeconv_native.edgeconv_forward(k, src.to(DEV), h_src.to(DEV), h_dst.to(DEV))
    assert arg.dtype == torch.int32
    assert torch.equal(arg.cpu(), ref_arg), "argmax indices differ"
    assert torch.equal(out.cpu(), ref_out), "max values are not bit-identical"


def test_edgeconv_backward_and_layer():
    from ae_mlsys_gnn_amd.layers import EdgeConv
    torch.manual_seed(0)
    bsz, npts, k = 2, 96, 20
    pts = torch.rand(bsz, npts, 3) * 2 - 1
    src = graphs.knn_graph(pts, k)
    x = pts.reshape(-1, 3)
    layer = EdgeConv(3, 64)
    # oracle: EdgeConv_reorg math in float64 with autograd (maxima are unique for random inputs)
    th = layer.theta.weight.detach().double().requires_grad_(True)
    ph = layer.phi.weight.detach().double().requires_grad_(True)
    xd = x.double()
    h_src = xd @ th.t()
    h_dst = xd @ ph.t() - h_src
    ref = orc.edgeconv_forward_autograd(k, src, h_src, h_dst)
    go = torch.randn(ref.shape, dtype=torch.float64)
    ref.backward(go)
    layer = layer.to(DEV)
    out = layer(k, src.to(DEV), x.to(DEV))
    out.backward(go.float().to(DEV))
    assert_close(out, ref.detach(), "edgeconv out")
    # the weight gradients are sums over the 192 points (and, for theta, the scattered neighbours) of terms
    # of either sign: bar from the sum of their absolute values
    _, arg = orc.edgeconv_forward(k, src, h_src.detach(), h_dst.detach())
    gsrc_abs = orc.edgeconv_backward(arg, go.abs(), xd.shape[0])[0]
    assert_close_sum(layer.theta.weight.grad, th.grad, (gsrc_abs + go.abs()).t() @ xd.abs(), "theta grad")
    assert_close_sum(layer.phi.weight.grad, ph.grad, go.abs().t() @ xd.abs(), "phi grad")


def test_edgeconv_backward_scatter_exact_counts():
    # grad_out = 1 makes the scatter-add an exact histogram of argmax: integer-valued, order independent
    from ae_mlsys_gnn_amd.operators.fused_edgeconv import edgeconv_native
    src, h_src, h_dst = _edgeconv_case(4, 256, 20, 3, 64, seed=5)
    out, arg = edgeconv_native.edgeconv_forward(20, src.to(DEV), h_src.to(DEV), h_dst.to(DEV))
    gs = edgeconv_native.edgeconv_backward(torch.ones_like(out), arg, h_src.shape[0])
    ref = c_oracle.edgeconv_backward(arg.cpu().numpy(), np.ones(out.shape), h_src.shape[0])
    assert np.array_equal(gs.cpu().numpy().astype(np.float64), ref)


# ------------------------------------------------------------------ GMMConv
def _gmm_case(g, k, dim, f, seed):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(g.n, k, f, generator=gen, dtype=torch.float64)
    pseudo = torch.rand(g.n_edges, dim, generator=gen, dtype=torch.float64)
    mu = torch.rand(k, dim, generator=gen, dtype=torch.float64)
    isg = 0.5 + torch.rand(k, dim, generator=gen, dtype=torch.float64)
    go = torch.randn(g.n, k, f, generator=gen, dtype=torch.float64)
    return x, pseudo, mu, isg, go


def _gmm_c(pseudo, mu, isg):
    """Constant of the derived bar for Gaussian weights: grows with the largest exponent magnitude."""
    v = 0.5 * (((pseudo.detach().double().unsqueeze(1) - mu.detach().double().unsqueeze(0)) * isg.detach().double().unsqueeze(0)) ** 2).sum(-1)
    return c_exp(float(v.max())) if v.numel() else c_exp(0.0)


def _gmm_check(got, want, g, x, pseudo, mu, isg, go, tag="", summed=False, shared=False):
    """(out, grad_feat, grad_pseudo, grad_mu, grad_sigma) against the oracle under the derived bar (rtol 1e-4 plus
    the rounding scale of each output's sum of absolute summands).  summed: the sum over the kernels is fused
    (out and go are [N,F]); shared: one [N,F] feature matrix serves all kernels."""
    k = mu.shape[0]
    xs = x.detach().unsqueeze(1).expand(-1, k, -1) if shared else x.detach()
    gs = go.unsqueeze(1).expand(-1, k, -1) if summed else go
    s = orc.gmm_abs_sums(g.row_ptr, g.col_ind, xs, pseudo.detach(), mu.detach(), isg.detach(), gs)
    scales = (s["out"].sum(1) if summed else s["out"], s["grad_feat"].sum(1) if shared else s["grad_feat"], s["grad_pseudo"],
              s["grad_mu"], s["grad_sigma"])
    c = _gmm_c(pseudo, mu, isg)
    for val, ref, sc, name in zip(got, want, scales, ("out", "grad node_feat", "grad pseudo", "grad mu", "grad inv_sigma")):
        if val is not None:
            assert_close_sum(val, ref, sc, "gmm " + name + tag, c=c)


@pytest.mark.parametrize("k,dim,f,variant", [(3, 2, 64, "fuse"), (2, 1, 16, "fuse"), (3, 2, 64, "stash"), (1, 3, 47, "fuse"),
                                              (4, 2, 33, "eb"), (3, 2, 128, "fuse"), (3, 2, 64, "sum"), (2, 3, 20, "sum"),
                                              (5, 2, 33, "sum"), (2, 1, 41, "fuse"), (9, 2, 5, "fuse"), (12, 1, 12, "sum"),
                                              # rows narrower than a wave: several edges per load instruction
                                              (1, 2, 8, "fuse"), (4, 2, 32, "fuse"), (1, 1, 128, "sum"), (2, 2, 32, "stash"), (2, 1, 16, "sum"),
                                              (3, 1, 4, "fuse"),
                                              # quarter of the width not a power of two: head-aligned lane map
                                              (2, 1, 44, "fuse"), (3, 2, 12, "sum"), (2, 2, 20, "stash"), (5, 1, 48, "fuse"), (4, 2, 100, "fuse"),
                                              (9, 1, 12, "fuse"),
                                              # summed kernels: lanes over F only, 1 to 64 rows per load instruction
                                              (3, 2, 4, "sum"), (4, 1, 8, "sum"), (2, 2, 256, "sum"), (4, 2, 128, "sum"), (1, 2, 44, "sum"),
                                              (3, 1, 100, "sum"), (2, 1, 252, "sum"), (4, 3, 32, "sum")])
def test_gmm_forward_backward(k, dim, f, variant, monkeypatch):
    from ae_mlsys_gnn_amd.operators import fused_gmmconv as fg
    from ae_mlsys_gnn_amd import _lib
    monkeypatch.setenv("FGNN_SEG_LEN", "256")
    _lib.clear_schedule_cache()
    g = graphs.add_csc_torch(degree_edge_graph(n=400, seed=k + f))
    x, pseudo, mu, isg, go = _gmm_case(g, k, dim, f, seed=1)
    leaves = [t.clone().requires_grad_(True) for t in (x, pseudo, mu, isg)]
    ref = orc.gmm_forward(g.row_ptr, g.col_ind, *leaves)
    ref.backward(go)
    gd = g.to(DEV)
    dl = [t.float().to(DEV).requires_grad_(True) for t in (x, pseudo, mu, isg)]
    op = {"fuse": fg.GmmConvFuse, "stash": fg.GmmConvStash, "eb": fg.GmmConvFuseEb, "sum": fg.GmmConvFuseSum}[variant]
    out = op(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, *dl)
    if variant == "sum":      # the sum over kernels fused into the operator: same gradients as summing outside
        for t in leaves:
            t.grad = None
        ref = orc.gmm_forward(g.row_ptr, g.col_ind, *leaves).sum(1)
        go = go[:, 0, :].contiguous()
        ref.backward(go)
    out.backward(go.float().to(DEV))
    _lib.clear_schedule_cache()
    _gmm_check((out, dl[0].grad, dl[1].grad, dl[2].grad, dl[3].grad), (ref.detach(),) + tuple(t.grad for t in leaves),
               g, x, pseudo, mu, isg, go, summed=variant == "sum")


@pytest.mark.parametrize("k,dim,f", [(2, 1, 16), (3, 2, 64), (4, 3, 32), (1, 1, 128), (2, 2, 256), (3, 2, 4), (2, 1, 44), (4, 1, 100), (1, 2, 8)])
def test_gmm_aggregate_shared_features(k, dim, f, monkeypatch):
    """GmmAggregate: one [N,F] feature matrix shared by the K mixture kernels (the aggregate-first form of the
    layers).  Oracle: the reference operator on the features repeated K times; its gradient summed over the
    copies.  Degrees 0..3000 with split rows, plain and XCD-aware schedules; unsupported shapes are refused."""
    from ae_mlsys_gnn_amd.operators import fused_gmmconv as fg
    from ae_mlsys_gnn_amd import _lib
    g = graphs.add_csc_torch(degree_edge_graph(n=400, seed=k + f))
    x, pseudo, mu, isg, go = _gmm_case(g, k, dim, f, seed=2)
    x = x[:, 0, :].contiguous()
    leaves = [t.clone().requires_grad_(True) for t in (x, pseudo, mu, isg)]
    ref = orc.gmm_forward(g.row_ptr, g.col_ind, leaves[0].unsqueeze(1).expand(-1, k, -1), *leaves[1:])
    ref.backward(go)
    gd = g.to(DEV)
    for buckets in ("0", "1"):
        monkeypatch.setenv("FGNN_SEG_LEN", "256")
        monkeypatch.setenv("FGNN_XCD_BUCKETS", buckets)
        monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
        _lib.clear_schedule_cache()
        dl = [t.float().to(DEV).requires_grad_(True) for t in (x, pseudo, mu, isg)]
        out = fg.GmmAggregate(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, *dl)
        assert out.shape == (g.n, k, f)
        out.backward(go.float().to(DEV))
        _gmm_check((out, dl[0].grad, dl[1].grad, dl[2].grad, dl[3].grad), (ref.detach(),) + tuple(t.grad for t in leaves),
                   g, x, pseudo, mu, isg, go, tag=" (aggregate, buckets %s)" % buckets, shared=True)
    _lib.clear_schedule_cache()
    # through the C ABI without a schedule (one wave per row)
    direct = torch.empty(g.n, k, f, device=DEV)
    dl = [t.float().to(DEV) for t in (x, pseudo, mu, isg)]
    _lib.check(_lib.lib().fgnn_gmm_forward(g.n, g.n_edges, k, dim, f, _lib.ptr(gd.row_ptr), _lib.ptr(gd.col_ind), None, _lib.ptr(dl[0]),
                                            _lib.ptr(dl[1]), _lib.ptr(dl[2]), _lib.ptr(dl[3]), _lib.ptr(direct), None, 2, None, None, 0,
                                            _lib.stream_ptr()), "fgnn_gmm_forward")
    torch.cuda.synchronize()
    _gmm_check((direct, None, None, None, None), (ref.detach(),) + tuple(t.grad for t in leaves), g, x, pseudo, mu, isg, go,
               tag=" (aggregate, no schedule)", shared=True)
    assert not fg.gmm_native.shared_supported(5, 16) and not fg.gmm_native.shared_supported(2, 18) and not fg.gmm_native.shared_supported(2, 260)
    with pytest.raises(_lib.FgnnError, match="shared node features"):
        fg.gmm_native.gmmconv_shared(gd.row_ptr, gd.col_ind, torch.zeros(g.n, 18, device=DEV), torch.zeros(g.n_edges, 1, device=DEV),
                                     torch.zeros(2, 1, device=DEV), torch.ones(2, 1, device=DEV))


@pytest.mark.parametrize("e,k,dim", [(1000, 3, 2), (1, 1, 1), (1025, 2, 1), (5000, 4, 3), (3000, 5, 2), (2049, 2, 4), (700, 7, 5)])
def test_gaussian_op(e, k, dim):
    """GaussianCp and its closed-form backward: mixtures with K <= 4, dim <= 3 take the kernel specialised at
    compile time (several edges per thread: edge counts around its 1024-edge blocks), the others the general one."""
    from ae_mlsys_gnn_amd.operators import fused_gmmconv as fg
    gen = torch.Generator().manual_seed(3 + e)
    pseudo = torch.rand(e, dim, generator=gen, dtype=torch.float64)
    mu = torch.rand(k, dim, generator=gen, dtype=torch.float64)
    isg = 0.5 + torch.rand(k, dim, generator=gen, dtype=torch.float64)
    go = torch.randn(e, k, generator=gen, dtype=torch.float64)
    leaves = [t.clone().requires_grad_(True) for t in (pseudo, mu, isg)]
    ref = orc.gaussian(*leaves)
    ref.backward(go)
    dl = [t.float().to(DEV).requires_grad_(True) for t in (pseudo, mu, isg)]
    out = fg.GaussianCp(*dl)
    out.backward(go.float().to(DEV))
    assert_close(out, ref.detach(), "gaussian")
    # closed-form derivatives, summed over k (pseudo) or over all edges (mu, sigma): scales = sums of |terms|
    t = (pseudo.unsqueeze(1) - mu.unsqueeze(0)).abs()
    gw = (go.abs() * ref.detach()).unsqueeze(-1)
    s2 = (isg ** 2).unsqueeze(0)
    c = _gmm_c(pseudo, mu, isg)
    assert_close_sum(dl[0].grad, leaves[0].grad, (gw * t * s2).sum(1), "grad pseudo", c=c)
    assert_close_sum(dl[1].grad, leaves[1].grad, (gw * t * s2).sum(0), "grad mu", c=c)
    assert_close_sum(dl[2].grad, leaves[2].grad, (gw * t * t * isg.unsqueeze(0)).sum(0), "grad sigma", c=c)


@pytest.mark.parametrize("fin,fout,k,dim,variant,agg_first", [(32, 16, 3, 2, "our", True), (32, 41, 2, 1, "our", True), (16, 24, 2, 1, "our", True),
                                                               (100, 16, 2, 1, "our", False), (30, 41, 2, 1, "our", False), (32, 7, 5, 2, "our", False),
                                                               (32, 7, 3, 2, "stash", False), (32, 16, 2, 3, "stash", False)])
def test_gmm_layer_matches_dgl_composed(fin, fout, k, dim, variant, agg_first):
    """Output and the gradients of the input, the pseudo-coordinates and every parameter against
    autograd through the float64 DGL-composed layer; odd widths go through the layer's zero padding.
    The recomputing layer aggregates its input before the fc when the input is narrower than K x out
    (and the operator takes the shape); the other cases transform first, as the reference does."""
    from ae_mlsys_gnn_amd.layers import GMMConv, GMMConv_stash
    torch.manual_seed(1)
    g = graphs.add_csc_torch(graphs.rmat_graph(500, 6000, seed=2))
    layer = (GMMConv if variant == "our" else GMMConv_stash)(fin, fout, dim=dim, n_kernels=k, residual=True, bias=True)
    with torch.no_grad():
        layer.bias.normal_()
    feat = torch.randn(g.n, fin)
    assert layer._aggregate_first(feat) == agg_first
    pseudo = torch.rand(g.n_edges, dim)
    go = torch.randn(g.n, fout)
    params = [layer.fc.weight, layer.mu, layer.inv_sigma, layer.bias, layer.res_fc.weight]
    leaves = [t.detach().double().requires_grad_(True) for t in params + [feat, pseudo]]
    ref = orc.gmm_layer_dgl(leaves[0], leaves[1], leaves[2], leaves[3], g.row_ptr, g.col_ind, leaves[5], leaves[6], leaves[4])
    ref.backward(go.double())
    gd = g.to(DEV)
    layer = layer.to(DEV)
    fd, pd = feat.to(DEV).requires_grad_(True), pseudo.to(DEV).requires_grad_(True)
    out = layer(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, fd, pd)
    assert out.shape == (g.n, fout)
    out.backward(go.to(DEV))
    # every output is a sum of terms of either sign (rows, then all nodes / edges for the parameters): derived bar
    d = [t.detach() for t in leaves]
    s = orc.gmm_layer_abs_sums(d[0], d[1], d[2], d[3], g.row_ptr, g.col_ind, d[5], d[6], d[4], go.double())
    c = _gmm_c(d[6], d[1], d[2])
    assert_close_sum(out, ref.detach(), s["out"], "GMMConv layer", c=c)
    assert_close_sum(fd.grad, leaves[5].grad, s["grad_feat"], "GMMConv grad feat", c=c)
    assert_close_sum(pd.grad, leaves[6].grad, s["grad_pseudo"], "GMMConv grad pseudo", c=c)
    for name, key, got, want in zip(("fc.weight", "mu", "inv_sigma", "bias", "res_fc.weight"), ("grad_fc", "grad_mu", "grad_sigma", "grad_bias", "grad_res"),
                                    (layer.fc.weight.grad, layer.mu.grad, layer.inv_sigma.grad, layer.bias.grad, layer.res_fc.weight.grad),
                                    (l.grad for l in leaves[:5])):
        assert_close_sum(got, want, s[key], "GMMConv grad " + name, c=c)


# ------------------------------------------------------------------ GAT layer vs the DGL-composed layer
@pytest.mark.parametrize("fin,f,h,variant", [(64, 16, 4, "our"), (30, 47, 1, "our"), (30, 47, 1, "stash"), (20, 6, 3, "fusescatter"),
                                             (12, 128, 1, "our")])
def test_gat_layer_matches_dgl_composed(fin, f, h, variant):
    """Output and the gradients of the input and of all three parameters against autograd through the
    float64 DGL-composed layer (config C1 graph); odd widths go through the layer's zero padding."""
    from ae_mlsys_gnn_amd.layers import GATConv, GATConv_fusescatter, GATConv_stash
    torch.manual_seed(2)
    g = graphs.add_csc_torch(graphs.uniform_graph(4096, 32768, seed=0))
    layer = {"our": GATConv, "stash": GATConv_stash, "fusescatter": GATConv_fusescatter}[variant](fin, f, h)
    feat = torch.randn(g.n, fin)
    go = torch.randn(g.n, h, f)
    # weight mapping to GATConv_dgl: fc.weight = W^T, attn_l(dgl) = attn_r(ours), attn_r(dgl) = attn_l(ours)
    leaves = [t.detach().double().requires_grad_(True) for t in (layer.W, layer.attn_l, layer.attn_r, feat)]
    ref = orc.gat_layer_dgl(leaves[0].t(), leaves[2], leaves[1], g.row_ptr, g.col_ind, 0.2, leaves[3])
    ref.backward(go.double())
    gd = g.to(DEV)
    layer = layer.to(DEV)
    fd = feat.to(DEV).requires_grad_(True)
    out = layer(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, fd, True if variant == "our" else gd.permute)
    assert out.shape == (g.n, h, f)
    out.backward(go.to(DEV))
    # projected features, outputs and gradients are all sums of terms of either sign (over the input width, the
    # neighbours, then the 4096 nodes for the parameters): derived bar from the sums of absolute summands
    d = [t.detach() for t in leaves]
    s = orc.gat_layer_abs_sums(d[0], d[1], d[2], g.row_ptr, g.col_ind, 0.2, d[3], go.double())
    hp = (d[3] @ d[0]).view(-1, h, f)
    c = c_exp(float((d[1] * hp).sum(-1).abs().max() + (d[2] * hp).sum(-1).abs().max()))
    assert_close_sum(out, ref.detach(), s["out"], "GATConv layer", c=c)
    assert_close_sum(fd.grad, leaves[3].grad, s["grad_feat"], "GATConv grad feat", c=c)
    assert_close_sum(layer.W.grad, leaves[0].grad, s["grad_W"], "GATConv grad W", c=c)
    assert_close_sum(layer.attn_l.grad, leaves[1].grad, s["grad_attn_l"], "GATConv grad attn_l", c=c)
    assert_close_sum(layer.attn_r.grad, leaves[2].grad, s["grad_attn_r"], "GATConv grad attn_r", c=c)
    # as a first layer (input without gradient: the backward reduces the two gradient parts separately)
    for p_ in layer.parameters():
        p_.grad = None
    out = layer(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, feat.to(DEV), True if variant == "our" else gd.permute)
    out.backward(go.to(DEV))
    assert_close_sum(out, ref.detach(), s["out"], "GATConv layer (first layer)", c=c)
    assert_close_sum(layer.W.grad, leaves[0].grad, s["grad_W"], "GATConv grad W (first layer)", c=c)
    assert_close_sum(layer.attn_l.grad, leaves[1].grad, s["grad_attn_l"], "GATConv grad attn_l (first layer)", c=c)
    assert_close_sum(layer.attn_r.grad, leaves[2].grad, s["grad_attn_r"], "GATConv grad attn_r (first layer)", c=c)


# ------------------------------------------------------------------ small operators
def _small_graph():
    return graphs.add_csc_torch(degree_edge_graph(n=300, seed=4))


@pytest.mark.parametrize("h,f", [(4, 16), (8, 32), (1, 47), (3, 20), (2, 128), (2, 41), (9, 5), (12, 12), (1, 4), (2, 8), (1, 128),
                                 (2, 44), (5, 48), (4, 100), (16, 12)])
def test_mhspmm_and_mhsddmm(h, f):
    from ae_mlsys_gnn_amd.operators import mhspmm as op
    g = _small_graph()
    gen = torch.Generator().manual_seed(h * f)
    feat = torch.randn(g.n, h, f, generator=gen, dtype=torch.float64)
    att = torch.randn(g.n_edges, h, generator=gen, dtype=torch.float64)
    go = torch.randn(g.n, h, f, generator=gen, dtype=torch.float64)
    fl, al = feat.clone().requires_grad_(True), att.clone().requires_grad_(True)
    ref = orc.mhspmm(g.row_ptr, g.col_ind, al, fl)
    ref.backward(go)
    gd = g.to(DEV)
    fd, ad = feat.float().to(DEV).requires_grad_(True), att.float().to(DEV).requires_grad_(True)
    out = op.csrmhspmm(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, fd, ad)
    out.backward(go.float().to(DEV))
    s_out, (s_att, s_feat) = orc.multilinear_abs_sums(lambda a, x: orc.mhspmm(g.row_ptr, g.col_ind, a, x), (att, feat), go)
    assert_close_sum(out, ref.detach(), s_out, "mhspmm")
    assert_close_sum(fd.grad, fl.grad, s_feat, "mhspmm grad feat")
    assert_close_sum(ad.grad, al.grad, s_att, "mhspmm grad att (mhsddmm)")
    tr = op.mhtranspose(gd.permute, ad.detach())
    assert torch.equal(tr.cpu(), att.float()[g.permute.long()])


# widths either side of the lane maps: 1, odd, powers of two, 33 (one entry per wave trip), 64, and 70 (the one-wave-per-row
# kernels); the graph has rows of 0..513 entries and a 3000-entry hub, so each width meets rows on both sides of the
# single-wave / whole-workgroup threshold
SMALL_OP_WIDTHS = [1, 3, 4, 8, 12, 33, 64, 70]


@pytest.mark.parametrize("nh", SMALL_OP_WIDTHS)
def test_edge_softmax(nh):
    from ae_mlsys_gnn_amd.operators import edge_softmax as op
    g = _small_graph()
    gen = torch.Generator().manual_seed(nh)
    h = torch.randn(g.n_edges, nh, generator=gen, dtype=torch.float64) * 3
    go = torch.randn(g.n_edges, nh, generator=gen, dtype=torch.float64)
    hl = h.clone().requires_grad_(True)
    ref = orc.edge_softmax(g.row_ptr, hl)
    ref.backward(go)
    hd = h.float().to(DEV).requires_grad_(True)
    out = op.csr_edge_softmax(g.row_ptr.to(DEV), hd)
    out.backward(go.float().to(DEV))
    assert_close(out, ref.detach(), "edge_softmax")
    assert_close(hd.grad, hl.grad, "edge_softmax grad")


@pytest.mark.parametrize("nh", SMALL_OP_WIDTHS)
def test_u_add_v(nh):
    from ae_mlsys_gnn_amd.operators import u_add_v as op
    g = _small_graph()
    gen = torch.Generator().manual_seed(100 + nh)
    rv = torch.randn(g.n, nh, generator=gen, dtype=torch.float64)
    cv = torch.randn(g.n, nh, generator=gen, dtype=torch.float64)
    go = torch.randn(g.n_edges, nh, generator=gen, dtype=torch.float64)
    rl, cl = rv.clone().requires_grad_(True), cv.clone().requires_grad_(True)
    ref = orc.u_add_v(g.row_ptr, g.col_ind, rl, cl)
    ref.backward(go)
    rd, cd = rv.float().to(DEV).requires_grad_(True), cv.float().to(DEV).requires_grad_(True)
    out = op.u_add_v_op(g.row_ptr.to(DEV), g.col_ind.to(DEV), rd, cd)
    out.backward(go.float().to(DEV))
    assert_close(out, ref.detach(), "u_add_v")
    _, (s_row, s_col) = orc.multilinear_abs_sums(lambda a, b: orc.u_add_v(g.row_ptr, g.col_ind, a, b), (rv, cv), go)
    assert_close_sum(rd.grad, rl.grad, s_row, "u_add_v grad row")
    assert_close_sum(cd.grad, cl.grad, s_col, "u_add_v grad col")


@pytest.mark.parametrize("w,max_deg", [(1, 6), (4, 6), (8, 6), (3, 8), (1, 22), (8, 22), (12, 30), (40, 3)])
def test_row_operators_where_short_rows_share_a_wave(w, max_deg):
    """Graphs whose mean row is a few entries (20 k rows of 0..max_deg entries, two long rows among them): the row kernels then
    give a row 8, 16 or 32 lanes and a wave takes several rows side by side.  Edge softmax both ways and both halves of the
    u_add_v backward (row sums, column sums) against float64; empty rows, rows past a group's registers and the long rows
    (which go to whole workgroups) included."""
    from ae_mlsys_gnn_amd.operators import edge_softmax as es
    from ae_mlsys_gnn_amd.operators import u_add_v as uav
    rng = np.random.default_rng(w * 100 + max_deg)
    n = 20000
    degs = rng.integers(0, max_deg + 1, size=n)
    degs[77] = 8192 // w + 5           # a long row (more than 8192 floats)
    degs[78] = 700                     # longer than any group's registers hold
    g = custom_graph([list(rng.integers(0, n, size=int(d))) for d in degs], n)
    gd = g.to(DEV)
    e = g.n_edges
    gen = torch.Generator().manual_seed(w + max_deg)
    x = torch.randn(e, w, generator=gen, dtype=torch.float64) * 2
    go = torch.randn(e, w, generator=gen, dtype=torch.float64)
    xl = x.clone().requires_grad_(True)
    ref = orc.edge_softmax(g.row_ptr, xl)
    ref.backward(go)
    xd = x.float().to(DEV).requires_grad_(True)
    out = es.csr_edge_softmax(gd.row_ptr, xd)
    out.backward(go.float().to(DEV))
    c = c_exp(float(x.max() - x.min()))
    one = torch.ones((), dtype=torch.float64)
    assert_close_sum(out, ref.detach(), one, "edge_softmax, short rows, width %d" % w, c=c)
    dst = orc.row_of_edge(g.row_ptr)
    dot_abs = orc.segment_sums(g.row_ptr, ref.detach() * go.abs())
    assert_close_sum(xd.grad, xl.grad, ref.detach() * (go.abs() + dot_abs[dst]), "edge_softmax grad, short rows, width %d" % w, c=c)
    rv = torch.randn(n, w, generator=gen, dtype=torch.float64)
    cv = torch.randn(n, w, generator=gen, dtype=torch.float64)
    rl, cl = rv.clone().requires_grad_(True), cv.clone().requires_grad_(True)
    orc.u_add_v(g.row_ptr, g.col_ind, rl, cl).backward(go)
    rd, cd = rv.float().to(DEV).requires_grad_(True), cv.float().to(DEV).requires_grad_(True)
    uav.u_add_v_op(gd.row_ptr, gd.col_ind, rd, cd).backward(go.float().to(DEV))
    _, (s_row, s_col) = orc.multilinear_abs_sums(lambda a, b: orc.u_add_v(g.row_ptr, g.col_ind, a, b), (rv, cv), go)
    assert_close_sum(rd.grad, rl.grad, s_row, "u_add_v grad row, short rows, width %d" % w)
    assert_close_sum(cd.grad, cl.grad, s_col, "u_add_v grad col, short rows, width %d" % w)


@pytest.mark.parametrize("seed", range(8))
def test_small_operators_on_random_heavy_tailed_graphs(seed):
    """Random graphs whose row lengths straddle the kernels' thresholds (empty rows, rows of a few entries, rows around
    8192 / width floats, one row of up to 12 k entries), random widths: edge softmax and u_add_v both ways, and the
    multi-head SDDMM, against the oracle."""
    from ae_mlsys_gnn_amd.operators import edge_softmax as es
    from ae_mlsys_gnn_amd.operators import mhspmm as mh
    from ae_mlsys_gnn_amd.operators import u_add_v as uav
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.integers(1, 300))
    w = int(rng.choice([1, 2, 4, 5, 8, 16, 24, 64]))
    edge = 8192 // w
    degs = rng.choice([0, 1, 3, 17, 64, edge - 1, edge, edge + 1, 2 * edge + 3], size=n, p=[.2, .2, .2, .15, .1, .04, .04, .04, .03])
    degs[int(rng.integers(0, n))] = int(rng.integers(3000, 12000))
    g = custom_graph([list(rng.integers(0, n, size=int(d))) for d in degs], n)
    gen = torch.Generator().manual_seed(seed)
    e = g.n_edges
    x = torch.randn(e, w, generator=gen, dtype=torch.float64) * 2
    go = torch.randn(e, w, generator=gen, dtype=torch.float64)
    xl = x.clone().requires_grad_(True)
    ref = orc.edge_softmax(g.row_ptr, xl)
    ref.backward(go)
    xd = x.float().to(DEV).requires_grad_(True)
    out = es.csr_edge_softmax(g.row_ptr.to(DEV), xd)
    out.backward(go.float().to(DEV))
    c = c_exp(float(x.max() - x.min()))
    one = torch.ones((), dtype=torch.float64)
    assert_close_sum(out, ref.detach(), one, "edge_softmax (random graph, width %d)" % w, c=c)
    dot_abs = orc.segment_sums(g.row_ptr, ref.detach() * go.abs())
    dst = orc.row_of_edge(g.row_ptr)
    assert_close_sum(xd.grad, xl.grad, ref.detach() * (go.abs() + dot_abs[dst]), "edge_softmax grad (random graph, width %d)" % w, c=c)
    rv = torch.randn(n, w, generator=gen, dtype=torch.float64)
    cv = torch.randn(n, w, generator=gen, dtype=torch.float64)
    rd, cd = rv.float().to(DEV).requires_grad_(True), cv.float().to(DEV).requires_grad_(True)
    o2 = uav.u_add_v_op(g.row_ptr.to(DEV), g.col_ind.to(DEV), rd, cd)
    o2.backward(go.float().to(DEV))
    assert torch.equal(o2.detach().cpu(), rv.float()[dst] + cv.float()[g.col_ind.long()])
    _, (s_row, s_col) = orc.multilinear_abs_sums(lambda a, b: orc.u_add_v(g.row_ptr, g.col_ind, a, b), (rv, cv), go)
    gl = [t.clone().requires_grad_(True) for t in (rv, cv)]
    orc.u_add_v(g.row_ptr, g.col_ind, *gl).backward(go)
    assert_close_sum(rd.grad, gl[0].grad, s_row, "u_add_v grad row (random graph)")
    assert_close_sum(cd.grad, gl[1].grad, s_col, "u_add_v grad col (random graph)")
    h, f = (w, 8) if w <= 16 else (4, 16)
    a = torch.randn(n, h, f, generator=gen, dtype=torch.float64)
    b = torch.randn(n, h, f, generator=gen, dtype=torch.float64)
    sd = mh.mhsddmm(g.row_ptr.to(DEV), g.col_ind.to(DEV), a.float().to(DEV), b.float().to(DEV))
    assert_close_sum(sd, orc.edge_dots(dst, g.col_ind.long(), a, b), orc.edge_dots(dst, g.col_ind.long(), a, b, absolute=True),
                     "mhsddmm (random graph)")


@pytest.mark.parametrize("weighted,sym", [(True, False), (False, False), (True, True)])
def test_csrspmm(weighted, sym):
    from ae_mlsys_gnn_amd.operators import spmm as op
    g = _small_graph()
    if sym:   # symmetric pattern: union of the graph and its transpose
        dst = orc.row_of_edge(g.row_ptr)
        src = g.col_ind.long()
        keys = torch.unique(torch.cat([dst * g.n + src, src * g.n + dst]))
        g = graphs.csr_from_keys(keys, g.n)
    x = torch.randn(g.n, 48, dtype=torch.float64)
    w = torch.rand(g.n_edges, dtype=torch.float64) if weighted else None
    if sym and weighted:   # symmetric values too
        dst = orc.row_of_edge(g.row_ptr)
        src = g.col_ind.long()
        w = torch.sin((dst + src).double()) + 0.1 * (dst * src % 7).double()
    go = torch.randn(g.n, 48, dtype=torch.float64)
    xl = x.clone().requires_grad_(True)
    wl = None if w is None else w.clone().requires_grad_(True)
    ref = orc.spmm(g.row_ptr, g.col_ind, xl, wl)
    ref.backward(go)
    xd = x.float().to(DEV).requires_grad_(True)
    wd = None if w is None else w.float().to(DEV).requires_grad_(True)
    out = op.csrspmm(g.row_ptr.to(DEV), g.col_ind.to(DEV), xd, wd, sym)
    out.backward(go.float().to(DEV))
    if weighted:
        s_out, (s_x, s_w) = orc.multilinear_abs_sums(lambda a, b: orc.spmm(g.row_ptr, g.col_ind, a, b), (x, w), go)
    else:
        s_out, (s_x,) = orc.multilinear_abs_sums(lambda a: orc.spmm(g.row_ptr, g.col_ind, a), (x,), go)
    assert_close_sum(out, ref.detach(), s_out, "csrspmm")
    assert_close_sum(xd.grad, xl.grad, s_x, "csrspmm grad x")
    if weighted:
        assert_close_sum(wd.grad, wl.grad, s_w, "csrspmm grad w")


def test_error_paths_return_codes_not_aborts():
    from ae_mlsys_gnn_amd._lib import FgnnError
    from ae_mlsys_gnn_amd.operators import fused_gat as fg
    g = graphs.add_csc_torch(graphs.uniform_graph(64, 256)).to(DEV)
    x = torch.randn(64, 2, 1028, device=DEV)       # more than 1024 floats per head
    a = torch.randn(64, 2, device=DEV)
    with pytest.raises(FgnnError, match="1024"):
        fg.fused_gat_op(a, a, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, 0.2, x)
    x = torch.randn(64, 8, 256, device=DEV)       # H*F = 2048: served in head groups, but only under a schedule
    a = torch.randn(64, 8, device=DEV)
    with pytest.raises(FgnnError, match="need a schedule"):
        fg.gat_native.gat_forward(a, a, g.row_ptr, g.col_ind, 0.2, x, use_schedule=False)
    with pytest.raises(FgnnError, match="GPU only"):
        fg.fused_gat_op(a.cpu(), a.cpu(), g.row_ptr.cpu(), g.col_ind.cpu(), g.col_ptr.cpu(), g.row_ind.cpu(), 0.2, x.cpu())
    with pytest.raises(FgnnError, match="int32"):
        fg.fused_gat_op(a, a, g.row_ptr.long(), g.col_ind, g.col_ptr, g.row_ind, 0.2, torch.randn(64, 8, 4, device=DEV))


@pytest.mark.parametrize("h,f", [(1, 64), (1, 47), (4, 16), (3, 20), (9, 5), (2, 256), (2, 44), (12, 12)])
def test_coo_and_csr_sddmm(h, f):
    """sddmm.coo_sddmm / csr_sddmm: per-edge dot products, against float64 gathers."""
    from ae_mlsys_gnn_amd.operators import sddmm
    g = _small_graph()
    gen = torch.Generator().manual_seed(h * 100 + f)
    e = 777                                                    # not a multiple of 64
    rows = torch.randint(0, g.n, (e,), generator=gen, dtype=torch.int32)
    cols = torch.randint(0, g.n, (e,), generator=gen, dtype=torch.int32)
    a = torch.randn(g.n, h, f, generator=gen, dtype=torch.float64)
    b = torch.randn(g.n, h, f, generator=gen, dtype=torch.float64)
    want = (a[rows.long()] * b[cols.long()]).sum(-1)
    got = sddmm.coo_sddmm(rows.to(DEV), cols.to(DEV), a.float().to(DEV), b.float().to(DEV))
    assert_close_sum(got, want, (a[rows.long()].abs() * b[cols.long()].abs()).sum(-1), "coo_sddmm")
    if h == 1:
        got1 = sddmm.coo_sddmm(rows.to(DEV), cols.to(DEV), a[:, 0].float().to(DEV), b[:, 0].float().to(DEV))
        assert torch.equal(got1, got[:, 0])
        dst = torch.repeat_interleave(torch.arange(g.n), (g.row_ptr[1:] - g.row_ptr[:-1]).long())
        want_csr = (a[dst, 0] * b[g.col_ind.long(), 0]).sum(-1)
        got_csr = sddmm.csr_sddmm(g.row_ptr.to(DEV), g.col_ind.to(DEV), a[:, 0].float().to(DEV), b[:, 0].float().to(DEV))
        assert_close_sum(got_csr, want_csr, (a[dst, 0].abs() * b[g.col_ind.long(), 0].abs()).sum(-1), "csr_sddmm")
    assert sddmm.coo_sddmm(rows[:0].to(DEV), cols[:0].to(DEV), a.float().to(DEV), b.float().to(DEV)).shape == (0, h)


# ------------------------------------------------------------------ kNN graph builder
@pytest.mark.parametrize("b,p,d,k", [(3, 100, 3, 5), (2, 1024, 3, 20), (2, 300, 64, 20), (1, 64, 7, 64), (4, 65, 2, 1),
                                     (2, 2500, 5, 70), (1, 1025, 9, 128), (2, 257, 11, 65), (3, 513, 1, 8)])
def test_knn_graph(b, p, d, k):
    from ae_mlsys_gnn_amd.operators.knn import knn_graph
    gen = torch.Generator().manual_seed(b * p + d)
    pts = torch.rand(b, p, d, generator=gen) * 2 - 1
    src = knn_graph(pts.to(DEV), k).cpu().long().view(b, p, k)
    # brute force in float64: exact squared distances
    dist = ((pts.double().unsqueeze(2) - pts.double().unsqueeze(1)) ** 2).sum(-1)          # [b,p,p]
    off = (torch.arange(b) * p).view(b, 1, 1)
    local = src - off
    assert bool(((local >= 0) & (local < p)).all()), "neighbours must stay inside their cloud"
    assert bool((local[:, :, 0] == torch.arange(p).view(1, p)).all()), "the nearest point is the point itself"
    got = torch.gather(dist, 2, local)
    want = torch.topk(dist, k, dim=2, largest=False).values
    # same k smallest distances, in ascending order (fp32 accumulation: tiny slack; ties may swap ids)
    assert bool((got[:, :, 1:] >= got[:, :, :-1] - 1e-6).all())
    assert float((got - want).abs().max()) < 1e-5
    assert all(torch.unique(local[i, j]).numel() == k for i in range(b) for j in range(0, p, 7)), "neighbours of a point are distinct"


def test_knn_graph_ties_are_ordered_by_id():
    """Integer grid coordinates: every squared distance is exact in fp32 and many are equal, so the
    neighbour ids themselves are fixed by the (distance, id) order."""
    from ae_mlsys_gnn_amd.operators.knn import knn_graph
    from ae_mlsys_gnn_amd._lib import FgnnError
    gen = torch.Generator().manual_seed(5)
    for (b, p, d, k) in [(2, 1500, 2, 40), (1, 300, 3, 100), (2, 64, 1, 64)]:
        pts = torch.randint(0, 12, (b, p, d), generator=gen).float()           # duplicates included
        src = knn_graph(pts.to(DEV), k).cpu().long().view(b, p, k)
        dist = ((pts.double().unsqueeze(2) - pts.double().unsqueeze(1)) ** 2).sum(-1)
        key = dist * p + torch.arange(p, dtype=torch.float64).view(1, 1, p)     # exact: dist < 2^10, p < 2^11
        want = torch.argsort(key, dim=2)[:, :, :k] + (torch.arange(b) * p).view(b, 1, 1)
        assert torch.equal(src, want), (b, p, d, k)
    with pytest.raises(FgnnError, match="128"):
        knn_graph(torch.zeros(1, 200, 3, device=DEV), 129)


def test_knn_graph_feeds_edgeconv():
    from ae_mlsys_gnn_amd.layers import EdgeConv
    from ae_mlsys_gnn_amd.operators.knn import knn_graph
    torch.manual_seed(0)
    pts = (torch.rand(4, 256, 3) * 2 - 1).to(DEV)
    src = knn_graph(pts, 20)
    layer = EdgeConv(3, 64).to(DEV)
    h = layer(20, src, pts.reshape(-1, 3))
    src2 = knn_graph(h.detach().view(4, 256, 64), 20)          # dynamic graph in feature space, as DGCNN does
    out = EdgeConv(64, 64).to(DEV)(20, src2, h)
    out.sum().backward()
    assert out.shape == (1024, 64) and bool(torch.isfinite(out).all())


@pytest.mark.parametrize("b,p,k,f,block", [(4, 256, 20, 64, 256), (3, 1000, 8, 20, 1000), (2, 2048, 10, 8, 2048), (5, 100, 5, 130, 100),
                                            (4, 256, 20, 64, 128), (4, 256, 20, 64, 1024), (2, 300, 6, 16, 8192)])
def test_edgeconv_backward_blocked(b, p, k, f, block):
    """The blocked backward (LDS tiles per cloud) against the oracle's scatter-add; block sizes that
    match the clouds, cut them in two, span several of them (overflow path) or exceed the LDS tile
    (fallback to the plain scatter)."""
    from ae_mlsys_gnn_amd.operators.fused_edgeconv import edgeconv_native
    from ae_mlsys_gnn_amd.operators.knn import knn_graph
    gen = torch.Generator().manual_seed(b * p + f)
    pts = (torch.rand(b, p, 3, generator=gen) * 2 - 1).to(DEV)
    src = knn_graph(pts, k)
    n = b * p
    hs, hd = torch.randn(n, f, generator=gen), torch.randn(n, f, generator=gen)
    go = torch.randn(n, f, generator=gen)
    out, arg = edgeconv_native.edgeconv_forward(k, src, hs.to(DEV), hd.to(DEV))
    want = torch.zeros(n, f, dtype=torch.float64).scatter_add_(0, arg.cpu().long(), go.double())
    got = edgeconv_native.edgeconv_backward(go.to(DEV), arg, n, block=block)
    s_abs = torch.zeros(n, f, dtype=torch.float64).scatter_add_(0, arg.cpu().long(), go.double().abs())
    assert_close_sum(got, want, s_abs, "blocked edgeconv backward")
    plain = edgeconv_native.edgeconv_backward(go.to(DEV), arg, n)
    assert_close_sum(plain, want, s_abs, "plain edgeconv backward")


def test_edgeconv_backward_blocked_with_a_wrong_hint():
    """Neighbours anywhere in the graph: every contribution outside a node's own block goes through the
    overflow list, the result is still the scatter-add."""
    from ae_mlsys_gnn_amd.operators.fused_edgeconv import fused_edgeconv_op
    gen = torch.Generator().manual_seed(3)
    n, k, f = 3000, 7, 24
    src = torch.randint(0, n, (n * k,), generator=gen, dtype=torch.int32)
    hs, hd, go = (torch.randn(n, f, generator=gen) for _ in range(3))
    ref_s = hs.double().requires_grad_(True)
    ref = orc.edgeconv_forward_autograd(k, src, ref_s, hd.double())
    ref.backward(go.double())
    hsd = hs.to(DEV).requires_grad_(True)
    out = fused_edgeconv_op(k, src.to(DEV), hsd, hd.to(DEV), block=512)
    out.backward(go.to(DEV))
    assert torch.equal(out.detach().cpu(), ref.detach().float())
    _, arg = orc.edgeconv_forward(k, src, hs.double(), hd.double())
    assert_close_sum(hsd.grad, ref_s.grad, orc.edgeconv_backward(arg, go.double().abs(), n)[0], "grad_src with a wrong block hint")


# ------------------------------------------------------------------ coo2csr (bit-exact)
@pytest.mark.parametrize("n,e,dedupe", [(1, 1, True), (50, 400, True), (50, 400, False), (3000, 200000, True), (70000, 500000, True), (300, 0, True)])
def test_coo2csr_bit_exact(n, e, dedupe):
    import scipy.sparse as sp
    from ae_mlsys_gnn_amd.operators import csr2csc as op
    gen = torch.Generator().manual_seed(n + e)
    # skewed endpoints so that duplicates are common
    dst = (torch.rand(e, generator=gen) ** 2 * n).long().clamp(max=n - 1).int()
    src = (torch.rand(e, generator=gen) ** 3 * n).long().clamp(max=n - 1).int()
    row_ptr, col_ind, edge_pos = op.coo2csr(dst.to(DEV), src.to(DEV), n, dedupe=dedupe, return_edge_pos=True)
    if dedupe:       # scipy merges duplicates (script/train/train_gatconv_our.py:87-91 relies on that)
        m = sp.csr_matrix((np.ones(e), (dst.numpy(), src.numpy())), shape=(n, n))
        m.sum_duplicates(); m.sort_indices()
        assert np.array_equal(row_ptr.cpu().numpy(), m.indptr) and np.array_equal(col_ind.cpu().numpy(), m.indices)
    else:
        order = np.lexsort((src.numpy(), dst.numpy()))
        assert np.array_equal(col_ind.cpu().numpy(), src.numpy()[order])
        assert np.array_equal(row_ptr.cpu().numpy(), np.concatenate([[0], np.cumsum(np.bincount(dst.numpy(), minlength=n))]))
    if e:
        # every input edge sits at its CSR position
        ep = edge_pos.cpu().long()
        rows = orc.row_of_edge(row_ptr.cpu())
        assert torch.equal(rows[ep], dst.long()) and torch.equal(col_ind.cpu().long()[ep], src.long())


def test_coo2csr_matches_graph_builder_at_scale():
    from ae_mlsys_gnn_amd.operators import csr2csc as op
    g = graphs.rmat_graph(100000, 4000000, seed=5, device=DEV)
    dst = torch.repeat_interleave(torch.arange(g.n, device=DEV, dtype=torch.int32), (g.row_ptr[1:] - g.row_ptr[:-1]).long())
    perm = torch.randperm(g.n_edges, device=DEV)
    d2 = torch.cat([dst[perm], dst[perm][:1000]])          # shuffled, with 1000 duplicated edges
    s2 = torch.cat([g.col_ind[perm], g.col_ind[perm][:1000]])
    row_ptr, col_ind = op.coo2csr(d2, s2, g.n)
    assert torch.equal(row_ptr, g.row_ptr) and torch.equal(col_ind, g.col_ind)


# ------------------------------------------------------------------ per-edge-array operators under XCD-aware schedules
def test_mhspmm_and_gmm_with_xcd_buckets(monkeypatch):
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.operators import fused_gmmconv as fg
    from ae_mlsys_gnn_amd.operators import mhspmm as op
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    monkeypatch.setenv("FGNN_SEG_LEN", "128")
    _lib.clear_schedule_cache()
    g = graphs.add_csc_torch(graphs.rmat_graph(1500, 120000, seed=12))
    gd = g.to(DEV)
    gen = torch.Generator().manual_seed(5)
    feat = torch.randn(g.n, 4, 16, generator=gen, dtype=torch.float64)
    att = torch.randn(g.n_edges, 4, generator=gen, dtype=torch.float64)
    go = torch.randn(g.n, 4, 16, generator=gen, dtype=torch.float64)
    fl, al = feat.clone().requires_grad_(True), att.clone().requires_grad_(True)
    ref = orc.mhspmm(g.row_ptr, g.col_ind, al, fl)
    ref.backward(go)
    fd, ad = feat.float().to(DEV).requires_grad_(True), att.float().to(DEV).requires_grad_(True)
    out = op.csrmhspmm(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, fd, ad)
    out.backward(go.float().to(DEV))
    s_out, (s_att, s_feat) = orc.multilinear_abs_sums(lambda a, x: orc.mhspmm(g.row_ptr, g.col_ind, a, x), (att, feat), go)
    assert_close_sum(out, ref.detach(), s_out, "mhspmm (buckets)")
    assert_close_sum(fd.grad, fl.grad, s_feat, "mhspmm grad feat (buckets)")
    assert_close_sum(ad.grad, al.grad, s_att, "mhspmm grad att (buckets)")
    # head counts that are multiples of four read the weights in place as 128-bit words; for others above two the wrapper's
    # workspace has room for the weights in the work list's entry order (copied there first, then streamed), and with a
    # workspace that only holds the partial results the same call reads them in place: same terms in the same order
    sch = _lib.schedule_for(gd.row_ptr, idx_tensor=gd.col_ind)
    assert sch.handle is not None
    assert _lib.lib().fgnn_mhspmm_workspace_bytes(sch.handle, 4, 16) == _lib.lib().fgnn_gmm_forward_workspace_bytes(sch.handle, 4, 16)
    assert _lib.lib().fgnn_mhspmm_workspace_bytes(sch.handle, 6, 16) > _lib.lib().fgnn_gmm_forward_workspace_bytes(sch.handle, 6, 16)
    for hh in (4, 6):
        a_h = torch.randn(g.n_edges, hh, generator=gen).to(DEV)
        x_h = torch.randn(g.n, hh, 16, generator=gen).to(DEV)
        want = orc.mhspmm(g.row_ptr, g.col_ind, a_h.cpu().double(), x_h.cpu().double())
        for pm in (None, gd.permute):
            ptr_arr, idx = (gd.row_ptr, gd.col_ind) if pm is None else (gd.col_ptr, gd.row_ind)
            sc = _lib.schedule_for(ptr_arr, idx_tensor=idx)
            copied = op.mhspmm(ptr_arr, idx, a_h, x_h, pos_map=pm)
            in_place = torch.empty_like(copied)
            ws, wsb = _lib.workspace(_lib.lib().fgnn_gmm_forward_workspace_bytes(sc.handle, hh, 16), DEV)
            _lib.check(_lib.lib().fgnn_mhspmm(g.n, g.n_edges, hh, 16, _lib.ptr(ptr_arr), _lib.ptr(idx), _lib.ptr(pm), _lib.ptr(a_h),
                                               _lib.ptr(x_h), _lib.ptr(in_place), sc.handle, _lib.ptr(ws), wsb, _lib.stream_ptr()), "fgnn_mhspmm")
            assert torch.equal(copied, in_place)
            if pm is None:
                assert_close_sum(copied, want, orc.mhspmm(g.row_ptr, g.col_ind, a_h.cpu().double().abs(), x_h.cpu().double().abs()),
                                 "mhspmm with %d heads under an XCD-aware list" % hh)
    # the SDDMM under the work list against the list-free kernel: the same dot product per entry, stored at the same place
    sd = op.mhsddmm(gd.row_ptr, gd.col_ind, go.float().to(DEV), fd.detach())
    plain = torch.empty_like(sd)
    _lib.check(_lib.lib().fgnn_mhsddmm(g.n, g.n_edges, 4, 16, _lib.ptr(gd.row_ptr), _lib.ptr(gd.col_ind), _lib.ptr(go.float().to(DEV).contiguous()),
                                        _lib.ptr(fd.detach()), _lib.ptr(plain), _lib.stream_ptr()), "fgnn_mhsddmm")
    assert torch.equal(sd, plain)
    for (k, dim, f) in [(3, 2, 64), (2, 1, 16)]:            # a full-width row and one narrower than a wave
        x, pseudo, mu, isg, go = _gmm_case(g, k, dim, f, seed=2)
        leaves = [t.clone().requires_grad_(True) for t in (x, pseudo, mu, isg)]
        ref = orc.gmm_forward(g.row_ptr, g.col_ind, *leaves)
        ref.backward(go)
        dl = [t.float().to(DEV).requires_grad_(True) for t in (x, pseudo, mu, isg)]
        out = fg.GmmConvStash(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, *dl)
        out.backward(go.float().to(DEV))
        _gmm_check((out, dl[0].grad, dl[1].grad, dl[2].grad, dl[3].grad), (ref.detach(),) + tuple(t.grad for t in leaves),
                   g, x, pseudo, mu, isg, go, tag=" (buckets)")
    _lib.clear_schedule_cache()


# ------------------------------------------------------------------ HIP graph capture of a launch-bound step
def test_edgeconv_step_replays_from_a_hip_graph():
    """EdgeConv forward + backward captured into a HIP graph (the library clears memory with fill
    kernels, never with memset nodes).  Every replay is checked against an eager run on fresh inputs,
    with eager work and synchronisations between the replays."""
    from ae_mlsys_gnn_amd.operators.fused_edgeconv import edgeconv_native
    from ae_mlsys_gnn_amd.operators.knn import knn_graph
    torch.manual_seed(3)
    n, f, k = 4 * 256, 64, 20
    pts = (torch.rand(4, 256, 3) * 2 - 1).to(DEV)
    src = knn_graph(pts, k)
    h_src = torch.randn(n, f, device=DEV)
    h_dst = torch.randn(n, f, device=DEV)
    go = torch.randn(n, f, device=DEV)
    # warm up on a side stream, then capture
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            out, arg = edgeconv_native.edgeconv_forward(k, src, h_src, h_dst)
            gs = edgeconv_native.edgeconv_backward(go, arg, n)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out, arg = edgeconv_native.edgeconv_forward(k, src, h_src, h_dst)
        gs = edgeconv_native.edgeconv_backward(go, arg, n)
    for rep in range(4):
        h_src.copy_(torch.randn(n, f, device=DEV))           # new inputs in the captured buffers
        h_dst.copy_(torch.randn(n, f, device=DEV))
        go.copy_(torch.round(torch.randn(n, f, device=DEV) * 8) / 8)     # dyadic values: the scatter sum is order independent
        graph.replay()
        torch.cuda.synchronize()
        e_out, e_arg = edgeconv_native.edgeconv_forward(k, src, h_src, h_dst)
        e_gs = edgeconv_native.edgeconv_backward(go, e_arg, n)
        torch.cuda.synchronize()
        assert torch.equal(out, e_out) and torch.equal(arg, e_arg), "replay %d: forward differs from eager" % rep
        assert torch.equal(gs, e_gs), "replay %d: backward differs from eager" % rep


@pytest.mark.parametrize("k,dim,f", [(3, 2, 16), (2, 1, 41), (2, 1, 16)])
def test_gmm_layer_with_csc_ordered_pseudo(k, dim, f, monkeypatch):
    """GMMConv(..., pseudo_csc=pseudo[permute]): same output; the gradient that arrives at pseudo_csc is
    the oracle's grad_pseudo in CSC order; all other gradients unchanged.  With an XCD-aware schedule too."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.layers import GMMConv
    for buckets in ("0", "1"):
        monkeypatch.setenv("FGNN_XCD_BUCKETS", buckets)
        monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
        _lib.clear_schedule_cache()
        torch.manual_seed(4)
        g = graphs.add_csc_torch(graphs.rmat_graph(600, 30000, seed=6))
        layer = GMMConv(24, f, dim=dim, n_kernels=k)
        feat, pseudo, go = torch.randn(g.n, 24), torch.rand(g.n_edges, dim), torch.randn(g.n, f)
        leaves = [t.detach().double().requires_grad_(True) for t in (layer.fc.weight, layer.mu, layer.inv_sigma, layer.bias, feat, pseudo)]
        ref = orc.gmm_layer_dgl(leaves[0], leaves[1], leaves[2], leaves[3], g.row_ptr, g.col_ind, leaves[4], leaves[5])
        ref.backward(go.double())
        gd = g.to(DEV)
        layer = layer.to(DEV)
        fd = feat.to(DEV).requires_grad_(True)
        pd = pseudo.to(DEV)
        pc = pd[gd.permute.long()].contiguous().requires_grad_(True)
        out = layer(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, fd, pd, pseudo_csc=pc)
        out.backward(go.to(DEV))
        d = [t.detach() for t in leaves]
        s = orc.gmm_layer_abs_sums(d[0], d[1], d[2], d[3], g.row_ptr, g.col_ind, d[4], d[5], None, go.double())
        c = _gmm_c(d[5], d[1], d[2])
        assert_close_sum(out, ref.detach(), s["out"], "GMMConv (two orders)", c=c)
        assert_close_sum(fd.grad, leaves[4].grad, s["grad_feat"], "grad feat (two orders)", c=c)
        assert_close_sum(pc.grad, leaves[5].grad[g.permute.long()], s["grad_pseudo"][g.permute.long()], "grad pseudo in CSC order", c=c)
        assert_close_sum(layer.mu.grad, leaves[1].grad, s["grad_mu"], "grad mu (two orders)", c=c)
        assert_close_sum(layer.inv_sigma.grad, leaves[2].grad, s["grad_sigma"], "grad inv_sigma (two orders)", c=c)
        assert_close_sum(layer.fc.weight.grad, leaves[0].grad, s["grad_fc"], "grad fc (two orders)", c=c)
    _lib.clear_schedule_cache()


@pytest.mark.parametrize("stash", [False, True])
@pytest.mark.parametrize("k,dim,f", [(3, 2, 16), (2, 1, 41), (2, 1, 16)])
def test_gmm_layer_with_pseudo_in_schedule_order(k, dim, f, stash, monkeypatch):
    """GMMConv(..., own_order=True) with the pseudo-coordinates permuted into the entry order of the
    operators' schedules (gmm_edge_positions): same output and gradients as the oracle, the gradient of
    the pseudo-coordinates arrives in the backward schedule's order.  XCD-aware (a real permutation) and
    plain schedules (identity, positions None); a forward-only call; asking for the positions twice."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.layers import GMMConv, GMMConv_stash
    from ae_mlsys_gnn_amd.operators.fused_gmmconv import gmm_edge_positions
    # 250 nodes: rows average 160 entries, both passes take an XCD-aware schedule; 600 nodes: 50 entries, the
    # summed backward keeps the caller's order there
    for buckets, n_nodes in (("1", 250), ("1", 600), ("0", 600)):
        monkeypatch.setenv("FGNN_XCD_BUCKETS", buckets)
        monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
        _lib.clear_schedule_cache()
        torch.manual_seed(4)
        g = graphs.add_csc_torch(graphs.rmat_graph(n_nodes, 30000 if n_nodes == 600 else 40000, seed=6))
        layer = (GMMConv_stash if stash else GMMConv)(24, f, dim=dim, n_kernels=k)      # the stash layer keeps the weights [E,K] as well
        feat, pseudo, go = torch.randn(g.n, 24), torch.rand(g.n_edges, dim), torch.randn(g.n, f)
        leaves = [t.detach().double().requires_grad_(True) for t in (layer.fc.weight, layer.mu, layer.inv_sigma, layer.bias, feat, pseudo)]
        ref = orc.gmm_layer_dgl(leaves[0], leaves[1], leaves[2], leaves[3], g.row_ptr, g.col_ind, leaves[4], leaves[5])
        ref.backward(go.double())
        gd = g.to(DEV)
        layer = layer.to(DEV)
        fd = feat.to(DEV).requires_grad_(True)
        pos_r, pos_c = gmm_edge_positions(gd.row_ptr, gd.col_ind), gmm_edge_positions(gd.col_ptr, gd.row_ind, summed_backward=True)
        assert (pos_r is None) == (buckets == "0") and (pos_c is None) == (buckets == "0" or n_nodes == 600)
        for pos, ptr_arr in ((pos_r, g.row_ptr), (pos_c, g.col_ptr)):        # a permutation that stays inside every row
            if pos is not None:
                assert torch.equal(pos.long().sort().values.cpu(), torch.arange(g.n_edges))
                row_of = torch.repeat_interleave(torch.arange(g.n), (ptr_arr[1:] - ptr_arr[:-1]).long())
                assert torch.equal(row_of[pos.long().cpu()], row_of)
                assert not torch.equal(pos.cpu(), torch.arange(g.n_edges, dtype=torch.int32))
        if pos_r is not None:
            assert torch.equal(gmm_edge_positions(gd.row_ptr, gd.col_ind), pos_r)           # asked again: same map
        identity = torch.arange(g.n_edges, device=DEV, dtype=torch.int32)
        pos_r, pos_c = identity if pos_r is None else pos_r, identity if pos_c is None else pos_c
        to_csc = gd.permute.long()[pos_c.long()]
        pd = pseudo.to(DEV)[pos_r.long()].contiguous()
        pc = pseudo.to(DEV)[to_csc].contiguous().requires_grad_(True)
        out = layer(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, fd, pd, pseudo_csc=pc, own_order=True)
        out.backward(go.to(DEV))
        d = [t.detach() for t in leaves]
        s = orc.gmm_layer_abs_sums(d[0], d[1], d[2], d[3], g.row_ptr, g.col_ind, d[4], d[5], None, go.double())
        c = _gmm_c(d[5], d[1], d[2])
        assert_close_sum(out, ref.detach(), s["out"], "GMMConv (schedule order)", c=c)
        assert_close_sum(fd.grad, leaves[4].grad, s["grad_feat"], "grad feat (schedule order)", c=c)
        assert_close_sum(pc.grad, leaves[5].grad[to_csc.cpu()], s["grad_pseudo"][to_csc.cpu()], "grad pseudo in the backward schedule's order", c=c)
        assert_close_sum(layer.mu.grad, leaves[1].grad, s["grad_mu"], "grad mu (schedule order)", c=c)
        assert_close_sum(layer.inv_sigma.grad, leaves[2].grad, s["grad_sigma"], "grad inv_sigma (schedule order)", c=c)
        assert_close_sum(layer.fc.weight.grad, leaves[0].grad, s["grad_fc"], "grad fc (schedule order)", c=c)
        with torch.no_grad():
            assert_close_sum(layer(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, fd, pd, own_order=True), ref.detach(),
                             s["out"], "GMMConv forward only (schedule order)", c=c)
        with pytest.raises(ValueError, match="forward-only"):
            layer(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, fd, pd, own_order=True)
    _lib.clear_schedule_cache()


def test_schedule_take_positions_c_abi(monkeypatch):
    """fgnn_schedule_take_positions: the map of an XCD-aware schedule is handed over once; a schedule built
    without positions refuses; a plain schedule returns the identity; afterwards mhspmm takes its per-edge
    weights in the schedule's order."""
    from ae_mlsys_gnn_amd import _lib
    g = graphs.rmat_graph(500, 20000, seed=9).to(DEV)
    s = _lib.Schedule(g.row_ptr, 0, g.col_ind, 16, with_positions=True)
    pos = s.take_positions()
    assert s.own_order and torch.equal(pos.long().sort().values.cpu(), torch.arange(g.n_edges))
    with pytest.raises(_lib.FgnnError, match="taken before"):
        s.take_positions()
    with pytest.raises(_lib.FgnnError, match="without edge positions"):
        _lib.Schedule(g.row_ptr, 0, g.col_ind, 16, with_positions=False).take_positions()
    plain = _lib.Schedule(g.row_ptr, 0)
    assert torch.equal(plain.take_positions().cpu(), torch.arange(g.n_edges, dtype=torch.int32))
    # the cached own-order schedule exists only after edge_positions was asked for
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    _lib.clear_schedule_cache()
    with pytest.raises(_lib.FgnnError, match="edge_positions"):
        _lib.schedule_for(g.row_ptr, idx_tensor=g.col_ind, own_order=True)
    again = _lib.edge_positions(g.row_ptr, g.col_ind)
    assert _lib.schedule_for(g.row_ptr, idx_tensor=g.col_ind, own_order=True).own_order
    assert _lib.schedule_for(g.row_ptr, idx_tensor=g.col_ind) is not _lib.schedule_for(g.row_ptr, idx_tensor=g.col_ind, own_order=True)
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    _lib.clear_schedule_cache()
    assert torch.equal(_lib.edge_positions(g.row_ptr, g.col_ind), pos) and again.numel() == g.n_edges
    _lib.clear_schedule_cache()
    # the operator under the own-order schedule: weights permuted by `pos` give the caller-order result
    torch.manual_seed(1)
    h, f = 2, 16
    x, w = torch.randn(g.n, h, f, device=DEV), torch.rand(g.n_edges, h, device=DEV)
    out = torch.empty(g.n, h, f, device=DEV)
    wo = w[pos.long()].contiguous()
    ws, wsb = _lib.workspace(_lib.lib().fgnn_mhspmm_workspace_bytes(s.handle, h, f), x.device)
    _lib.check(_lib.lib().fgnn_mhspmm(g.n, g.n_edges, h, f, _lib.ptr(g.row_ptr), _lib.ptr(g.col_ind), None, _lib.ptr(wo), _lib.ptr(x),
                                       _lib.ptr(out), s.handle, _lib.ptr(ws), wsb, _lib.stream_ptr()), "fgnn_mhspmm")
    torch.cuda.synchronize()
    want = orc.mhspmm(g.row_ptr.cpu(), g.col_ind.cpu(), w.cpu().double(), x.cpu().double())
    assert_close_sum(out, want, orc.mhspmm(g.row_ptr.cpu(), g.col_ind.cpu(), w.cpu().double(), x.cpu().double().abs()),
                     "mhspmm under an own-order schedule")


@pytest.mark.parametrize("d", [1, 2, 3, 4])
@pytest.mark.parametrize("e", [1, 257, 300001])
def test_edge_linear_tanh_matches_torch(d, e):
    """Linear(2, d) + Tanh over the edges (the MoNet drivers' pseudo projection): forward and the
    parameter gradients against torch in float64; the gradient sums are reproducible run to run."""
    from ae_mlsys_gnn_amd.operators import edge_proj
    torch.manual_seed(d * 1000 + e)
    x = torch.rand(e, 2, dtype=torch.float64) * 2 - 1
    w = torch.randn(d, 2, dtype=torch.float64, requires_grad=True)
    b = torch.randn(d, dtype=torch.float64, requires_grad=True)
    go = torch.randn(e, d, dtype=torch.float64)
    want = torch.tanh(torch.nn.functional.linear(x, w, b))
    want.backward(go)
    xd = x.float().to(DEV)
    wd = w.detach().float().to(DEV).requires_grad_(True)
    bd = b.detach().float().to(DEV).requires_grad_(True)
    got = edge_proj.edge_linear_tanh(xd, wd, bd)
    got.backward(go.float().to(DEV))
    assert_close(got, want, "y")
    # sums over the e edges of terms of either sign: derived bar from the sums of their absolute values
    gt = (go * (1 - want.detach() ** 2)).abs()
    assert_close_sum(wd.grad, w.grad, gt.t() @ x.abs(), "grad_W")
    assert_close_sum(bd.grad, b.grad, gt.sum(0), "grad_b")
    w2 = wd.detach().clone().requires_grad_(True)
    b2 = bd.detach().clone().requires_grad_(True)
    edge_proj.edge_linear_tanh(xd, w2, b2).backward(go.float().to(DEV))
    assert torch.equal(w2.grad, wd.grad) and torch.equal(b2.grad, bd.grad)


def test_edge_linear_tanh_limits():
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.operators import edge_proj
    with pytest.raises(ValueError):
        edge_proj.edge_linear_tanh(torch.rand(5, 2, device=DEV), torch.rand(5, 2, device=DEV), torch.rand(5, device=DEV))
    assert _lib.lib().fgnn_edge_linear_tanh(4, 5, None, None, None, None, None) == -4
    y = edge_proj.edge_linear_tanh(torch.rand(0, 2, device=DEV), torch.rand(2, 2, device=DEV), torch.rand(2, device=DEV))
    assert y.shape == (0, 2)


@pytest.mark.parametrize("b,p,k,fin,f,block,slope", [(3, 128, 10, 3, 64, 128, 0.2), (2, 100, 7, 5, 20, None, 0.2), (2, 256, 20, 3, 130, 256, 0.01),
                                                       (4, 64, 5, 8, 8, 32, 1.0)])
def test_edgeconv_with_fused_leaky_relu(b, p, k, fin, f, block, slope):
    """EdgeConv(..., negative_slope_out=s) == LeakyReLU(s)(EdgeConv(...)) (script/train/train_edgeconv_our.py:56):
    outputs bit-identical to the unfused pair on the GPU and equal to the float64 oracle's; gradients of theta and
    phi against autograd through the oracle (plain and blocked backward, the mask replayed from the output)."""
    from ae_mlsys_gnn_amd.layers import EdgeConv
    torch.manual_seed(b * p + f)
    pts = torch.rand(b, p, 3) * 2 - 1
    src = graphs.knn_graph(pts, k)
    x = torch.randn(b * p, fin)
    layer = EdgeConv(fin, f)
    th = layer.theta.weight.detach().double().requires_grad_(True)
    ph = layer.phi.weight.detach().double().requires_grad_(True)
    xd = x.double().requires_grad_(True)
    h_src = xd @ th.t()
    h_dst = xd @ ph.t() - h_src
    ref = torch.nn.functional.leaky_relu(orc.edgeconv_forward_autograd(k, src, h_src, h_dst), slope)
    go = torch.randn(ref.shape, dtype=torch.float64)
    ref.backward(go)
    layer = layer.to(DEV)
    xg = x.to(DEV).requires_grad_(True)
    out = layer(k, src.to(DEV), xg, block=block, negative_slope_out=slope)
    out.backward(go.float().to(DEV))
    unfused = torch.nn.functional.leaky_relu(layer(k, src.to(DEV), x.to(DEV), block=block), slope)
    assert torch.equal(out.detach(), unfused.detach()), "fused activation is not bit-identical to the unfused pair"
    assert_close(out, ref.detach(), "edgeconv + lrelu out")
    # scales of the weight / input gradients: sums over points (and scattered neighbours) of |masked gradient| |x|
    _, arg = orc.edgeconv_forward(k, src, h_src.detach(), h_dst.detach())
    gm = (go * torch.where(ref.detach() > 0, 1.0, slope)).abs()
    gsrc_abs = orc.edgeconv_backward(arg, gm, xd.shape[0])[0]
    assert_close_sum(layer.theta.weight.grad, th.grad, (gsrc_abs + gm).t() @ xd.detach().abs(), "theta grad")
    assert_close_sum(layer.phi.weight.grad, ph.grad, gm.t() @ xd.detach().abs(), "phi grad")
    assert_close_sum(xg.grad, xd.grad, (gsrc_abs + gm) @ th.detach().abs() + gm @ ph.detach().abs(), "input grad")
    from ae_mlsys_gnn_amd._lib import FgnnError
    with pytest.raises(FgnnError, match="positive"):
        layer(k, src.to(DEV), x.to(DEV), negative_slope_out=0.0)


@pytest.mark.parametrize("k,dim,f,with_bias,with_res", [(3, 2, 64, True, True), (2, 1, 16, True, False), (4, 2, 32, False, True), (2, 2, 256, True, True),
                                                         (3, 1, 44, True, True)])
def test_gmm_sum_with_bias_and_residual_in_the_store(k, dim, f, with_bias, with_res, monkeypatch):
    """GmmConvFuseSum(..., bias, residual): the rest of the layer's forward (layers/gmmconv_layer.py:69-75 of the
    reference) added inside the operator's store, whole rows and merged split rows, plain and XCD-aware work lists;
    output and every gradient (bias and residual included) against the float64 oracle."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.operators import fused_gmmconv as fg
    g = graphs.add_csc_torch(degree_edge_graph(n=400, seed=k + f))
    x, pseudo, mu, isg, go = _gmm_case(g, k, dim, f, seed=3)
    go = go[:, 0, :].contiguous()
    gen = torch.Generator().manual_seed(9)
    bias = torch.randn(f, generator=gen, dtype=torch.float64) if with_bias else None
    res = torch.randn(g.n, f, generator=gen, dtype=torch.float64) if with_res else None
    leaves = [t.clone().requires_grad_(True) for t in (x, pseudo, mu, isg)]
    bl = None if bias is None else bias.clone().requires_grad_(True)
    rl = None if res is None else res.clone().requires_grad_(True)
    ref = orc.gmm_forward(g.row_ptr, g.col_ind, *leaves).sum(1)
    if rl is not None:
        ref = ref + rl
    if bl is not None:
        ref = ref + bl
    ref.backward(go)
    gd = g.to(DEV)
    for buckets in ("0", "1"):
        monkeypatch.setenv("FGNN_SEG_LEN", "256")
        monkeypatch.setenv("FGNN_XCD_BUCKETS", buckets)
        monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
        _lib.clear_schedule_cache()
        dl = [t.float().to(DEV).requires_grad_(True) for t in (x, pseudo, mu, isg)]
        bd = None if bias is None else bias.float().to(DEV).requires_grad_(True)
        rd = None if res is None else res.float().to(DEV).requires_grad_(True)
        out = fg.GmmConvFuseSum(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, *dl, bias=bd, residual=rd)
        out.backward(go.float().to(DEV))
        s = orc.gmm_abs_sums(g.row_ptr, g.col_ind, x, pseudo, mu, isg, go.unsqueeze(1).expand(-1, k, -1))
        s_out = s["out"].sum(1) + (0 if res is None else res.abs()) + (0 if bias is None else bias.abs())
        c = _gmm_c(pseudo, mu, isg)
        assert_close_sum(out, ref.detach(), s_out, "out with epilogue (buckets %s)" % buckets, c=c)
        for val, want, key in zip((t.grad for t in dl), (t.grad for t in leaves), ("grad_feat", "grad_pseudo", "grad_mu", "grad_sigma")):
            assert_close_sum(val, want, s[key], key + " with epilogue", c=c)
        if bd is not None:
            assert_close_sum(bd.grad, bl.grad, go.abs().sum(0), "grad bias")
        if rd is not None:
            assert torch.equal(rd.grad.cpu(), go.float())
    _lib.clear_schedule_cache()
    with pytest.raises(_lib.FgnnError, match="sum over the kernels"):
        fg.gmm_native.gmmconv(gd.row_ptr, gd.col_ind, dl[0].detach(), dl[1].detach(), dl[2].detach(), dl[3].detach(), bias=torch.zeros(f, device=DEV))


# ------------------------------------------------------------------ column sums under a tile-ordered plan
@pytest.mark.parametrize("w,lds,task_len", [(1, 1024, 64), (3, 1024, 0), (4, 2048, 100), (8, 0, 0), (8, 4096, 256), (12, 1024, 64),
                                            (33, 4096, 0), (64, 8192, 300), (128, 16384, 0), (256, 65536, 64)])
def test_edge_colsum_under_a_plan(w, lds, task_len):
    """out[j] = sum of g[p] over the entries of column j: rectangular pattern (more columns than rows, the last range
    partly filled), unsorted rows with repeated columns, empty columns, ranges cut into several tasks and merged; against
    float64, twice with equal bits, and through fgnn_u_add_v_backward_planned on the square pattern."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.operators.u_add_v import u_add_v_native
    rng = np.random.default_rng(w * 7 + lds)
    n_rows, n_cols = 257, 1500
    rows = []
    for i in range(n_rows):
        d = int(rng.choice([0, 1, 5, 40, 700]))
        cols = rng.integers(0, n_cols - 300, size=d)          # the last 300 columns stay empty
        rows.append(list(np.sort(cols)) if i % 3 else list(cols))
    g = custom_graph(rows, n_rows)
    e = g.n_edges
    gen = torch.Generator().manual_seed(w)
    val = torch.randn(e, w, generator=gen)
    ref = torch.zeros(n_cols, w, dtype=torch.float64).index_add_(0, g.col_ind.long(), val.double())
    s_abs = torch.zeros(n_cols, w, dtype=torch.float64).index_add_(0, g.col_ind.long(), val.double().abs())
    rp, ci, vd = g.row_ptr.to(DEV), g.col_ind.to(DEV), val.to(DEV)
    plan = _lib.ColsumPlan(rp, ci, n_cols, w, lds_bytes=lds, task_len=task_len)
    assert plan.n_tasks >= (n_cols + plan.columns_per_range - 1) // plan.columns_per_range
    out = plan.colsum(vd)
    assert_close_sum(out, ref, s_abs, "edge colsum W=%d" % w)
    assert torch.equal(out, plan.colsum(vd)), "column sums differ between two runs"
    if w > 1:          # a plan serves narrower arrays
        out1 = plan.colsum(vd[:, :1].contiguous())
        assert_close_sum(out1, ref[:, :1], s_abs[:, :1], "edge colsum W=1 under a plan for W=%d" % w)
    # the square pattern through the u_add_v backward, both forms
    sq = custom_graph([[c % n_rows for c in r] for r in rows], n_rows)
    rp2, ci2 = sq.row_ptr.to(DEV), sq.col_ind.to(DEV)
    ref_col = torch.zeros(n_rows, w, dtype=torch.float64).index_add_(0, sq.col_ind.long(), val.double())
    abs_col = torch.zeros(n_rows, w, dtype=torch.float64).index_add_(0, sq.col_ind.long(), val.double().abs())
    ref_row = orc.segment_sums(sq.row_ptr, val.double())
    abs_row = orc.segment_sums(sq.row_ptr, val.double().abs())
    for atomics in (False, True):
        grow, gcol = u_add_v_native.u_add_v_backward(rp2, ci2, vd, atomics=atomics)
        assert_close_sum(grow, ref_row, abs_row, "u_add_v grad row W=%d atomics=%s" % (w, atomics))
        assert_close_sum(gcol, ref_col, abs_col, "u_add_v grad col W=%d atomics=%s" % (w, atomics))


def test_edge_colsum_plan_argument_errors():
    from ae_mlsys_gnn_amd import _lib
    g = _small_graph().to(DEV)
    with pytest.raises(_lib.FgnnError, match="lds_bytes"):
        _lib.ColsumPlan(g.row_ptr, g.col_ind, g.n, 8, lds_bytes=100)
    with pytest.raises(_lib.FgnnError, match="too wide"):
        _lib.ColsumPlan(g.row_ptr, g.col_ind, g.n, 300, lds_bytes=1024)
    with pytest.raises(_lib.FgnnError, match="outside"):
        _lib.ColsumPlan(g.row_ptr, g.col_ind, g.n - 50, 8)          # column ids beyond n_cols
    plan = _lib.ColsumPlan(g.row_ptr, g.col_ind, g.n, 4, lds_bytes=65536)
    with pytest.raises(_lib.FgnnError, match="narrower"):
        plan.colsum(torch.zeros(g.n_edges, 64, device=DEV))
    empty = custom_graph([[] for _ in range(10)], 10).to(DEV)
    pe = _lib.ColsumPlan(empty.row_ptr, empty.col_ind, 10, 8)
    assert torch.equal(pe.colsum(torch.zeros(0, 8, device=DEV)), torch.zeros(10, 8, device=DEV))


@pytest.mark.parametrize("w", [1, 3, 4, 8, 12, 100, 512, 2051, 2052])
def test_gather_rows_widths(w):
    """mhtranspose for row widths on every side of the kernel's cases: scalar and 128-bit lanes, several rows per wave,
    one row per wave in one or several trips."""
    from ae_mlsys_gnn_amd.operators import mhspmm as op
    e = 777 if w < 512 else 37
    gen = torch.Generator().manual_seed(w)
    x = torch.randn(e, w, generator=gen)
    perm = torch.randperm(e, generator=gen).to(torch.int32)
    out = op.mhtranspose(perm.to(DEV), x.to(DEV))
    assert torch.equal(out.cpu(), x[perm.long()])
    # an unaligned view takes the scalar path
    if w % 4 == 0:
        buf = torch.randn(e * w + 1, generator=gen).to(DEV)
        xin = buf[1:].view(e, w)
        out = torch.empty(e * w + 1, device=DEV)[1:].view(e, w)
        from ae_mlsys_gnn_amd._lib import check, lib, ptr, stream_ptr
        check(lib().fgnn_gather_rows(e, w, ptr(perm.to(DEV)), ptr(xin), ptr(out), stream_ptr()), "fgnn_gather_rows")
        assert torch.equal(out.cpu(), xin.cpu()[perm.long()])


@pytest.mark.parametrize("n_short", [0, 6000, 60000])
@pytest.mark.parametrize("nh", [1, 4, 8, 20])
def test_edge_softmax_rows_beyond_the_register_cache(nh, n_short):
    """Rows longer than what a workgroup keeps in registers (the part beyond is folded into a running maximum and sum while
    it streams by): a 40 k-entry row whose values ascend, so the running maximum moves on every trip, one whose values
    descend, a constant one, next to short rows; forward and backward against float64.  With n_short rows of two entries
    appended the mean row is short and the launch takes its small-footprint configuration (fewer values cached, more
    streamed) for the same long rows; with 60000 of them the short rows share waves (groups of 8, 16 or 32 lanes per
    row, by head count)."""
    from ae_mlsys_gnn_amd.operators import edge_softmax as op
    lens = [40000, 3, 0, 40000, 9000, 1, 40000] + [2] * n_short
    g = custom_graph([[0] * d for d in lens], len(lens))
    e = g.n_edges
    gen = torch.Generator().manual_seed(nh)
    h = torch.randn(e, nh, generator=gen, dtype=torch.float64)
    ramp = torch.linspace(-30, 30, 40000, dtype=torch.float64).view(-1, 1)
    h[:40000] += ramp
    h[40003:80003] -= ramp
    h[89004:] = 1.5
    go = torch.randn(e, nh, generator=gen, dtype=torch.float64)
    hl = h.clone().requires_grad_(True)
    ref = orc.edge_softmax(g.row_ptr, hl)
    ref.backward(go)
    hd = h.float().to(DEV).requires_grad_(True)
    out = op.csr_edge_softmax(g.row_ptr.to(DEV), hd)
    out.backward(go.float().to(DEV))
    c = c_exp(float(h.max() - h.min()))
    one = torch.ones((), dtype=torch.float64)
    assert_close_sum(out, ref.detach(), one, "edge_softmax of long rows", c=c)
    dst = orc.row_of_edge(g.row_ptr)
    dot_abs = orc.segment_sums(g.row_ptr, ref.detach() * go.abs())
    assert_close_sum(hd.grad, hl.grad, ref.detach() * (go.abs() + dot_abs[dst]), "edge_softmax grad of long rows", c=c)
    sums = orc.segment_sums(g.row_ptr, out.detach().cpu().double())
    assert float((sums - (torch.tensor(lens) > 0).double().view(-1, 1)).abs().max()) < 1e-5
    assert (e * nh >= 1024 * len(lens)) == (n_short == 0)          # the two configurations' side of the mean-row-length rule


@pytest.mark.parametrize("h,f", [(8, 256), (3, 501), (5, 300)])
def test_mhspmm_and_mhsddmm_rows_wider_than_1024_floats(h, f, monkeypatch):
    """Head-group passes over views of the wide arrays (row stride H*F, shifted base), with and without an XCD-aware list."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.operators import mhspmm as op
    for buckets in ("0", "1"):
        monkeypatch.setenv("FGNN_XCD_BUCKETS", buckets)
        monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
        monkeypatch.setenv("FGNN_SEG_LEN", "256")
        _lib.clear_schedule_cache()
        g = graphs.add_csc_torch(degree_edge_graph(n=60, seed=81))
        gen = torch.Generator().manual_seed(h * f)
        feat = torch.randn(g.n, h, f, generator=gen, dtype=torch.float64)
        att = torch.randn(g.n_edges, h, generator=gen, dtype=torch.float64)
        go = torch.randn(g.n, h, f, generator=gen, dtype=torch.float64)
        fl, al = feat.clone().requires_grad_(True), att.clone().requires_grad_(True)
        ref = orc.mhspmm(g.row_ptr, g.col_ind, al, fl)
        ref.backward(go)
        gd = g.to(DEV)
        fd, ad = feat.float().to(DEV).requires_grad_(True), att.float().to(DEV).requires_grad_(True)
        out = op.csrmhspmm(gd.row_ptr, gd.col_ind, gd.col_ptr, gd.row_ind, gd.permute, fd, ad)
        out.backward(go.float().to(DEV))
        s_out, (s_att, s_feat) = orc.multilinear_abs_sums(lambda a, x: orc.mhspmm(g.row_ptr, g.col_ind, a, x), (att, feat), go)
        assert_close_sum(out, ref.detach(), s_out, "mhspmm, wide rows, buckets " + buckets)
        assert_close_sum(fd.grad, fl.grad, s_feat, "mhspmm grad feat, wide rows, buckets " + buckets)
        assert_close_sum(ad.grad, al.grad, s_att, "mhspmm grad att (mhsddmm), wide rows, buckets " + buckets)
    _lib.clear_schedule_cache()

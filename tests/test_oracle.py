"""Pins the CPU oracle (oracle/) without a GPU: every oracle function is checked against
something it was not written from -- dense brute force, closed forms, scipy, python loops, and
the independent plain-C restatement -- chosen so that a dropped term, a wrong sign or a swapped
src/dst fails at least one check."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from oracle import c_oracle
from oracle import fgnn_oracle as orc
from tests.util import custom_graph, degree_edge_graph, gat_inputs
from ae_mlsys_gnn_amd import graphs


def _close(a, b, tol=1e-10):
    a = torch.as_tensor(np.asarray(a)).double()
    b = torch.as_tensor(np.asarray(b)).double()
    assert a.shape == b.shape
    assert float((a - b).abs().max()) <= tol * max(1.0, float(b.abs().max())), float((a - b).abs().max())


# ------------------------------------------------------------------ GAT forward
@pytest.mark.parametrize("seed,slope", [(0, 0.2), (1, 0.01), (2, 1.0)])
def test_gat_forward_vs_dense_masked_softmax(seed, slope):
    g = graphs.uniform_graph(40, 300, seed=seed)
    x, ar, ac, _ = gat_inputs(g, 3, 5, seed)
    _close(orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, slope, x),
           orc.gat_forward_dense(ar, ac, g.row_ptr, g.col_ind, slope, x))


def test_gat_forward_vs_c_oracle_with_duplicates_and_empty_rows():
    g = degree_edge_graph(n=120, seed=3)     # duplicate edges, empty rows, a hub
    x, ar, ac, _ = gat_inputs(g, 2, 7, 1)
    out, e, alpha, mx, sm = orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x, return_edge=True)
    c_out, c_mx, c_sm = c_oracle.gat_forward(g.row_ptr, g.col_ind, ar, ac, 0.2, x)
    _close(out, c_out)
    deg = (g.row_ptr[1:] - g.row_ptr[:-1])
    nz = deg > 0
    _close(mx[nz], c_mx[nz.numpy()])
    _close(sm[nz], c_sm[nz.numpy()])
    assert np.all(c_out[~nz.numpy()] == 0) and np.all(c_mx[~nz.numpy()] == -1e38) and np.all(c_sm[~nz.numpy()] == 0)


def test_gat_closed_forms():
    g = graphs.rmat_graph(80, 700, seed=4)
    x, ar, ac, _ = gat_inputs(g, 2, 4, 2)
    # attention rows sum to one: constant features come back unchanged
    one = torch.ones_like(x)
    _close(orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, one), one)
    # zero attention: neighbour mean == row-normalised scipy SpMM
    z = torch.zeros_like(ar)
    a = sp.csr_matrix((np.ones(g.n_edges), g.col_ind.numpy(), g.row_ptr.numpy()), shape=(g.n, g.n))
    a = sp.diags(1.0 / np.asarray(a.sum(1)).ravel()) @ a
    _close(orc.gat_forward(z, z, g.row_ptr, g.col_ind, 0.2, x).reshape(g.n, -1), a @ x.reshape(g.n, -1).numpy())
    # only self loops: identity (graph of the reference's script/inference/gatconv_test.py:75-76)
    s = custom_graph([[0], [1], [2], [3]])
    xs, ars, acs, _ = gat_inputs(s, 2, 3, 0)
    _close(orc.gat_forward(ars, acs, s.row_ptr, s.col_ind, 0.2, xs), xs)
    # a destination-side score shift does not change a softmax when slope == 1
    _close(orc.gat_forward(ar + 3.0, ac, g.row_ptr, g.col_ind, 1.0, x), orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, 1.0, x))
    # ... but a source-side shift on ONE node does: src/dst are not interchangeable
    ac2 = ac.clone(); ac2[5] += 2.0
    assert float((orc.gat_forward(ar, ac2, g.row_ptr, g.col_ind, 1.0, x) - orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, 1.0, x)).abs().max()) > 1e-3


def test_gat_relabelling_invariance():
    g = graphs.uniform_graph(50, 400, seed=5)
    x, ar, ac, _ = gat_inputs(g, 2, 3, 3)
    perm = torch.randperm(g.n, generator=torch.Generator().manual_seed(1))     # new id of old node i is perm[i]
    dst = orc.row_of_edge(g.row_ptr)
    keys = torch.unique(perm[dst] * g.n + perm[g.col_ind.long()])
    g2 = graphs.csr_from_keys(keys, g.n)
    inv = torch.argsort(perm)
    out = orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, 0.2, x)
    out2 = orc.gat_forward(ar[inv], ac[inv], g2.row_ptr, g2.col_ind, 0.2, x[inv])
    _close(out2[perm], out)


def test_gat_layer_orientation_maps_to_dgl_layer():
    g = graphs.uniform_graph(60, 500, seed=6)
    gen = torch.Generator().manual_seed(0)
    w = torch.randn(10, 8, generator=gen, dtype=torch.float64)
    al = torch.randn(1, 2, 4, generator=gen, dtype=torch.float64)
    ar_ = torch.randn(1, 2, 4, generator=gen, dtype=torch.float64)
    feat = torch.randn(g.n, 10, generator=gen, dtype=torch.float64)
    ours = orc.gat_layer_ours(w, al, ar_, g.row_ptr, g.col_ind, 0.2, feat)
    _close(ours, orc.gat_layer_dgl(w.t(), ar_, al, g.row_ptr, g.col_ind, 0.2, feat))
    # un-swapped attention vectors give a different layer
    assert float((ours - orc.gat_layer_dgl(w.t(), al, ar_, g.row_ptr, g.col_ind, 0.2, feat)).abs().max()) > 1e-3


# ------------------------------------------------------------------ GAT backward
@pytest.mark.parametrize("slope", [0.2, 1.0])
def test_gat_backward_autograd_vs_analytic_c(slope):
    g = degree_edge_graph(n=90, seed=7)
    x, ar, ac, go = gat_inputs(g, 2, 5, 4)
    xl, al, cl = (t.clone().requires_grad_(True) for t in (x, ar, ac))
    orc.gat_forward(al, cl, g.row_ptr, g.col_ind, slope, xl).backward(go)
    gx, gar, gac = c_oracle.gat_backward(g.row_ptr, g.col_ind, ar, ac, slope, x, go)
    _close(xl.grad, gx)
    _close(al.grad, gar, 1e-9)
    _close(cl.grad, gac, 1e-9)
    if slope == 1.0:      # sum_p alpha_p (ge_p - ws) == 0 per row
        assert float(al.grad.abs().max()) < 1e-9


def test_gat_backward_identities_used_by_the_kernels():
    # delta = <g_out, out> and grad_attn_row = <g_out, out2> - delta*c with out2 = sum alpha*lrelu'*x
    g = graphs.rmat_graph(70, 600, seed=8)
    slope = 0.2
    x, ar, ac, go = gat_inputs(g, 2, 4, 5)
    out, e, alpha, _, _ = orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, slope, x, return_edge=True)
    dst = orc.row_of_edge(g.row_ptr); src = g.col_ind.long()
    lp = torch.where(e > 0, torch.ones_like(e), torch.full_like(e, slope))
    out2 = torch.zeros_like(x).index_add_(0, dst, (alpha * lp).unsqueeze(-1) * x[src])
    c = torch.zeros_like(ar).index_add_(0, dst, alpha * lp)
    delta = (go * out).sum(-1)
    al = ar.clone().requires_grad_(True)
    orc.gat_forward(al, ac, g.row_ptr, g.col_ind, slope, x).backward(go)
    _close((go * out2).sum(-1) - delta * c, al.grad, 1e-9)


# ------------------------------------------------------------------ EdgeConv
def test_edgeconv_vs_python_loops_with_ties():
    gen = torch.Generator().manual_seed(0)
    n, k, f = 30, 6, 5
    src = torch.randint(0, n, (n * k,), generator=gen, dtype=torch.int32)
    hs = torch.round(torch.randn(n, f, generator=gen))      # integers: many exact ties
    hd = torch.round(torch.randn(n, f, generator=gen))
    out, arg = orc.edgeconv_forward(k, src, hs, hd)
    for i in range(n):
        for c in range(f):
            best, ba = None, None
            for t in range(k):
                j = int(src[i * k + t])
                v = np.float32(hd[i, c].item()) + np.float32(hs[j, c].item())
                if best is None or v > best:
                    best, ba = v, j
            assert out[i, c].item() == best and arg[i, c].item() == ba
    c_out, c_arg = c_oracle.edgeconv_forward(k, src.numpy(), hs.numpy(), hd.numpy())
    assert np.array_equal(c_out, out.numpy()) and np.array_equal(c_arg, arg.numpy())
    # first maximum == the index torch.max reports on [n,k,f]
    v = hd.unsqueeze(1) + hs[src.long().view(n, k)]
    assert torch.equal(out, v.max(1).values)


def test_edgeconv_backward_scatter():
    gen = torch.Generator().manual_seed(1)
    n, k, f = 40, 5, 6
    src = torch.randint(0, n, (n * k,), generator=gen, dtype=torch.int32)
    hs = torch.randn(n, f, generator=gen, dtype=torch.float64).requires_grad_(True)
    hd = torch.randn(n, f, generator=gen, dtype=torch.float64).requires_grad_(True)
    go = torch.randn(n, f, generator=gen, dtype=torch.float64)
    orc.edgeconv_forward_autograd(k, src, hs, hd).backward(go)
    _, arg = orc.edgeconv_forward(k, src, hs.detach(), hd.detach())
    gs, gd = orc.edgeconv_backward(arg, go, n)
    _close(gs, hs.grad); _close(gd, hd.grad)
    _close(c_oracle.edgeconv_backward(arg.numpy(), go.numpy(), n), hs.grad)


def test_edgeconv_reorg_equals_unreorganised_form():
    # max_j theta(x_j - x_i) + phi(x_i) == max_j theta(x_j) + (phi - theta)(x_i) for bias-free maps
    gen = torch.Generator().manual_seed(2)
    n, k = 50, 4
    x = torch.randn(n, 3, generator=gen, dtype=torch.float64)
    th = torch.randn(8, 3, generator=gen, dtype=torch.float64); ph = torch.randn(8, 3, generator=gen, dtype=torch.float64)
    src = torch.randint(0, n, (n * k,), generator=gen, dtype=torch.int32)
    out, _ = orc.edgeconv_forward(k, src, x @ th.t(), x @ ph.t() - x @ th.t())
    xi = x.unsqueeze(1); xj = x[src.long().view(n, k)]
    _close(out, ((xj - xi) @ th.t() + (xi @ ph.t())).max(1).values, 1e-12)


# ------------------------------------------------------------------ GMMConv
def test_gmm_special_cases_and_c_oracle():
    g = graphs.rmat_graph(60, 500, seed=9)
    gen = torch.Generator().manual_seed(3)
    k, dim, f = 3, 2, 4
    x = torch.randn(g.n, k, f, generator=gen, dtype=torch.float64)
    ps = torch.rand(g.n_edges, dim, generator=gen, dtype=torch.float64)
    mu = torch.rand(k, dim, generator=gen, dtype=torch.float64)
    sg = 0.5 + torch.rand(k, dim, generator=gen, dtype=torch.float64)
    # inv_sigma == 0: every weight is 1, the op is a plain SpMM
    a = sp.csr_matrix((np.ones(g.n_edges), g.col_ind.numpy(), g.row_ptr.numpy()), shape=(g.n, g.n))
    _close(orc.gmm_forward(g.row_ptr, g.col_ind, x, ps, mu, torch.zeros_like(sg)).reshape(g.n, -1), a @ x.reshape(g.n, -1).numpy())
    # one edge, hand-computed weight
    w = orc.gaussian(torch.tensor([[0.5, 1.0]], dtype=torch.float64), torch.tensor([[0.0, 0.0]], dtype=torch.float64),
                     torch.tensor([[2.0, 1.0]], dtype=torch.float64))
    assert abs(w.item() - np.exp(-0.5 * (1.0 + 1.0))) < 1e-15
    _close(orc.gmm_forward(g.row_ptr, g.col_ind, x, ps, mu, sg), c_oracle.gmm_forward(g.row_ptr, g.col_ind, x, ps, mu, sg))
    go = torch.randn(g.n, k, f, generator=gen, dtype=torch.float64)
    leaves = [t.clone().requires_grad_(True) for t in (x, ps, mu, sg)]
    orc.gmm_forward(g.row_ptr, g.col_ind, *leaves).backward(go)
    gx, gp, gm, gs = c_oracle.gmm_backward(g.row_ptr, g.col_ind, x, ps, mu, sg, go)
    _close(leaves[0].grad, gx); _close(leaves[1].grad, gp, 1e-9); _close(leaves[2].grad, gm, 1e-9); _close(leaves[3].grad, gs, 1e-9)


def test_gmm_layer_dgl_reduces_to_scipy_spmm():
    """K = 1 and inv_sigma = 0 (every Gaussian weight is 1), no bias, no residual: the layer of
    layers/gmmconv_layer.py:130-149 is A @ (feat @ W.T) with A the 0/1 adjacency."""
    g = graphs.rmat_graph(70, 600, seed=12)
    gen = torch.Generator().manual_seed(5)
    fin, fout = 6, 5
    feat = torch.randn(g.n, fin, generator=gen, dtype=torch.float64)
    w = torch.randn(fout, fin, generator=gen, dtype=torch.float64)
    ps = torch.rand(g.n_edges, 2, generator=gen, dtype=torch.float64)
    mu = torch.rand(1, 2, generator=gen, dtype=torch.float64)
    a = sp.csr_matrix((np.ones(g.n_edges), g.col_ind.numpy(), g.row_ptr.numpy()), shape=(g.n, g.n))
    _close(orc.gmm_layer_dgl(w, mu, torch.zeros(1, 2, dtype=torch.float64), None, g.row_ptr, g.col_ind, feat, ps),
           a @ (feat.numpy() @ w.numpy().T))


def test_gmm_layer_dgl_hand_built_with_residual_bias_and_view_order():
    """3 nodes, 4 edges, K = 2, out = 2, dim = 1, worked out with python loops and math.exp.  Kernel k
    uses rows [k*out, (k+1)*out) of fc.weight (the `view(-1, K, out)` of layers/gmmconv_layer.py:133);
    reading the same fc output as (out, K) gives another number, so a swapped view cannot pass."""
    import math
    rows = [[1, 2], [0], [2]]                       # destination -> sources, CSR order
    g = custom_graph(rows)
    kk, fout, fin = 2, 2, 2
    feat = [[1.0, 2.0], [0.5, -1.0], [-2.0, 0.25]]
    wfc = [[1.0, 0.0], [0.0, 1.0], [2.0, -1.0], [0.5, 0.5]]          # [K*out, in]
    wres = [[0.1, 0.2], [-0.3, 0.4]]
    bias = [0.5, -0.25]
    pseudo = [0.2, 0.9, 0.4, 0.7]                   # one coordinate per CSR position
    mu = [0.1, 0.8]
    isg = [2.0, 0.5]

    def layer(view_k_major=True):
        out = [[0.0] * fout for _ in range(3)]
        pos = 0
        for i, srcs in enumerate(rows):
            for j in srcs:
                fc = [sum(wfc[r][c] * feat[j][c] for c in range(fin)) for r in range(kk * fout)]
                for k in range(kk):
                    wgt = math.exp(-0.5 * ((pseudo[pos] - mu[k]) * isg[k]) ** 2)
                    for o in range(fout):
                        out[i][o] += wgt * (fc[k * fout + o] if view_k_major else fc[o * kk + k])
                pos += 1
            for o in range(fout):
                out[i][o] += sum(wres[o][c] * feat[i][c] for c in range(fin)) + bias[o]
        return out

    t = lambda v: torch.tensor(v, dtype=torch.float64)
    got = orc.gmm_layer_dgl(t(wfc), t(mu).view(kk, 1), t(isg).view(kk, 1), t(bias), g.row_ptr, g.col_ind, t(feat),
                            t(pseudo).view(-1, 1), t(wres))
    _close(got, layer(True), 1e-14)
    assert float((got - t(layer(False))).abs().max()) > 0.1
    # residual and bias really are added: dropping either changes every row
    no_res = orc.gmm_layer_dgl(t(wfc), t(mu).view(kk, 1), t(isg).view(kk, 1), t(bias), g.row_ptr, g.col_ind, t(feat), t(pseudo).view(-1, 1))
    no_bias = orc.gmm_layer_dgl(t(wfc), t(mu).view(kk, 1), t(isg).view(kk, 1), None, g.row_ptr, g.col_ind, t(feat), t(pseudo).view(-1, 1), t(wres))
    _close(got - no_res, t(feat) @ t(wres).t(), 1e-14)
    _close(got - no_bias, t(bias).view(1, -1).expand(3, -1), 1e-14)


# ------------------------------------------------------------------ the error-bound scales (sums of |summands|)
def test_abs_sums_equal_outputs_for_non_negative_inputs_and_bound_them_otherwise():
    g = graphs.rmat_graph(60, 500, seed=13)
    x, ar, ac, go = gat_inputs(g, 2, 4, 5)
    slope = 0.2
    # slope = 1 and non-negative features / gradients: forward sums have no cancellation, so S == output
    s = orc.gat_abs_sums(ar, ac, g.row_ptr, g.col_ind, 1.0, x.abs(), go.abs())
    xr = x.abs().clone().requires_grad_(True)
    out = orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, 1.0, xr)
    out.backward(go.abs())
    _close(s["out"], out.detach()); _close(s["grad_feat"], xr.grad)
    # general signs: S bounds |output| for every output, and is strictly larger somewhere
    leaves = [t.clone().requires_grad_(True) for t in (ar, ac, x)]
    out = orc.gat_forward(leaves[0], leaves[1], g.row_ptr, g.col_ind, slope, leaves[2])
    out.backward(go)
    s = orc.gat_abs_sums(ar, ac, g.row_ptr, g.col_ind, slope, x, go)
    for name, val in (("out", out.detach()), ("grad_feat", leaves[2].grad), ("grad_attn_row", leaves[0].grad), ("grad_attn_col", leaves[1].grad)):
        assert bool((s[name] >= val.abs() - 1e-12).all()), name
        assert float((s[name] - val.abs()).max()) > 1e-3, name
    # GMM: with x, g >= 0 the forward and grad_feat sums are cancellation-free; t >= 0 when pseudo >= mu
    k, dim, f = 2, 2, 3
    gen = torch.Generator().manual_seed(6)
    xm = torch.rand(g.n, k, f, generator=gen, dtype=torch.float64)
    gm = torch.rand(g.n, k, f, generator=gen, dtype=torch.float64)
    ps = 1.0 + torch.rand(g.n_edges, dim, generator=gen, dtype=torch.float64)
    mu = torch.rand(k, dim, generator=gen, dtype=torch.float64)
    sg = 0.5 + torch.rand(k, dim, generator=gen, dtype=torch.float64)
    lv = [t.clone().requires_grad_(True) for t in (xm, ps, mu, sg)]
    o = orc.gmm_forward(g.row_ptr, g.col_ind, *lv)
    o.backward(gm)
    sm = orc.gmm_abs_sums(g.row_ptr, g.col_ind, xm, ps, mu, sg, gm)
    _close(sm["out"], o.detach()); _close(sm["grad_feat"], lv[0].grad)
    _close(sm["grad_mu"], lv[2].grad.abs(), 1e-9); _close(sm["grad_sigma"], lv[3].grad.abs(), 1e-9); _close(sm["grad_pseudo"], lv[1].grad.abs(), 1e-9)


@pytest.mark.parametrize("chunk", [5, 64, 1 << 20])
def test_gat_reference_chunked_equals_autograd_oracle(chunk):
    """The chunked float64 form used at full size (no [E,H,F] tensor, analytic backward) against gat_forward +
    autograd and gat_abs_sums; the graph has empty rows, a hub and duplicate edges, the chunks cut rows."""
    g = graphs.add_csc_torch(degree_edge_graph(n=90, seed=8))
    x, ar, ac, go = gat_inputs(g, 2, 5, 6)
    for slope in (0.2, 1.0):
        leaves = [t.clone().requires_grad_(True) for t in (ar, ac, x)]
        out = orc.gat_forward(leaves[0], leaves[1], g.row_ptr, g.col_ind, slope, leaves[2])
        out.backward(go)
        s = orc.gat_abs_sums(ar, ac, g.row_ptr, g.col_ind, slope, x, go)
        r = orc.gat_reference_chunked(ar.float(), ac.float(), g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute, slope, x.float(), go.float(),
                                      chunk=chunk)
        for name, want in (("out", out.detach()), ("grad_feat", leaves[2].grad), ("grad_attn_row", leaves[0].grad), ("grad_attn_col", leaves[1].grad)):
            _close(r[name], want, 1e-6)              # inputs went through float32
            _close(r["S_" + name], s[name], 1e-6)
        assert float(r["A_grad_attn_row"].abs().max()) == 0.0 and float(r["A_grad_attn_col"].abs().max()) == 0.0
    # a pre-activation of exactly zero (attn_row[i] == -attn_col[j]) is a point where LeakyReLU' jumps: the edge's
    # possible contribution shows up as an allowance on its row and its column, nowhere else
    i, j = 3, int(g.col_ind[int(g.row_ptr[3])])
    ar2 = ar.float().clone(); ar2[i, 0] = -ac.float()[j, 0]
    r = orc.gat_reference_chunked(ar2, ac.float(), g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute, 0.2, x.float(), go.float())
    assert float(r["A_grad_attn_row"][i, 0]) > 0 and float(r["A_grad_attn_col"][j, 0]) > 0
    assert int((r["A_grad_attn_row"] != 0).sum()) == 1


# ------------------------------------------------------------------ csr2csc
@pytest.mark.parametrize("seed", [0, 1])
def test_csr2csc_vs_scipy_bruteforce_and_c(seed):
    g = degree_edge_graph(n=150, seed=seed)          # duplicates, unsorted columns, empty rows/columns
    rp, ci = g.row_ptr.numpy(), g.col_ind.numpy()
    cp, ri, pm = orc.csr2csc(rp, ci)
    b = orc.csr2csc_bruteforce(rp, ci)
    c = c_oracle.csr2csc(rp, ci)
    for x, y, z in zip((cp, ri, pm), b, c):
        assert np.array_equal(x, y) and np.array_equal(x, z)
    # scipy (what the reference scripts use, script/train/train_gmmconv_our.py:80-93) on a duplicate-free graph
    g2 = graphs.rmat_graph(200, 3000, seed=seed)
    rp, ci = g2.row_ptr.numpy(), g2.col_ind.numpy()
    m = sp.csr_matrix((np.arange(g2.n_edges, dtype=np.int64), ci, rp), shape=(g2.n, g2.n)).tocsc()
    cp, ri, pm = orc.csr2csc(rp, ci)
    assert np.array_equal(cp, m.indptr) and np.array_equal(ri, m.indices) and np.array_equal(pm, m.data)


# ------------------------------------------------------------------ small operators
def test_small_ops_vs_scipy_and_loops():
    g = graphs.rmat_graph(50, 400, seed=10)
    gen = torch.Generator().manual_seed(4)
    rp, ci = g.row_ptr.numpy(), g.col_ind.numpy()
    x = torch.randn(g.n, 6, generator=gen, dtype=torch.float64)
    w = torch.rand(g.n_edges, generator=gen, dtype=torch.float64)
    a = sp.csr_matrix((w.numpy(), ci, rp), shape=(g.n, g.n))
    _close(orc.spmm(g.row_ptr, g.col_ind, x, w), a @ x.numpy())
    _close(orc.mhspmm(g.row_ptr, g.col_ind, w.view(-1, 1), x.view(g.n, 1, 6)).reshape(g.n, 6), a @ x.numpy())
    y = torch.randn(g.n, 6, generator=gen, dtype=torch.float64)
    d = (x.numpy() @ y.numpy().T)
    rows = np.repeat(np.arange(g.n), np.diff(rp))
    _close(orc.sddmm(g.row_ptr, g.col_ind, x, y), d[rows, ci])
    _close(orc.mhsddmm(g.row_ptr, g.col_ind, x.view(g.n, 2, 3), y.view(g.n, 2, 3))[:, 1],
           np.einsum("ef,ef->e", x.view(g.n, 2, 3).numpy()[rows, 1], y.view(g.n, 2, 3).numpy()[ci, 1]))
    _close(orc.u_add_v(g.row_ptr, g.col_ind, x, y), x.numpy()[rows] + y.numpy()[ci])
    h = torch.randn(g.n_edges, 2, generator=gen, dtype=torch.float64)
    s = orc.edge_softmax(g.row_ptr, h)
    for i in range(g.n):
        seg = slice(rp[i], rp[i + 1])
        _close(s[seg], torch.softmax(h[seg], 0))


# ------------------------------------------------------------------ golden fixtures stay in step with the oracle
def test_golden_fixtures_match_oracle():
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    d = np.load(os.path.join(here, "gat_rmat_h4f16.npz"))
    out = orc.gat_forward(torch.from_numpy(d["attn_row"]).double(), torch.from_numpy(d["attn_col"]).double(),
                          torch.from_numpy(d["row_ptr"]), torch.from_numpy(d["col_ind"]), float(d["slope"]), torch.from_numpy(d["x"]).double())
    _close(out, d["out"])
    c_out, _, _ = c_oracle.gat_forward(d["row_ptr"], d["col_ind"], d["attn_row"], d["attn_col"], float(d["slope"]), d["x"])
    _close(c_out, d["out"])
    gx, gar, gac = c_oracle.gat_backward(d["row_ptr"], d["col_ind"], d["attn_row"], d["attn_col"], float(d["slope"]), d["x"], d["grad_out"])
    _close(gx, d["grad_x"]); _close(gar, d["grad_attn_row"], 1e-9); _close(gac, d["grad_attn_col"], 1e-9)
    e = np.load(os.path.join(here, "edgeconv_k20_f64.npz"))
    c_out, c_arg = c_oracle.edgeconv_forward(int(e["k"]), e["src_ind"], e["h_src"], e["h_dst"])
    assert np.array_equal(c_out, e["out"]) and np.array_equal(c_arg, e["argmax"])
    m = np.load(os.path.join(here, "gmm_k3_d2_f16.npz"))
    _close(c_oracle.gmm_forward(m["row_ptr"], m["col_ind"], m["x"], m["pseudo"], m["mu"], m["inv_sigma"]), m["out"])
    cp, ri, pm = c_oracle.csr2csc(m["row_ptr"], m["col_ind"])
    assert np.array_equal(cp, m["col_ptr"]) and np.array_equal(ri, m["row_ind"]) and np.array_equal(pm, m["permute"])

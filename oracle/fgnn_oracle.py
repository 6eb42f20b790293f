"""CPU oracle for the fused GNN sparse-operator path (TEST INFRASTRUCTURE ONLY).

This module restates, in plain torch on the CPU, the layer math that the reference
composes out of DGL message-passing primitives, plus dense brute-force forms for
tiny graphs.  It is the *checker*: only tests, the smoke entry and the CPU-baseline
leg of the benchmark may import it.  Nothing in the shipped package does.

Index convention (reference script/train/train_gatconv_our.py:87-91): CSR rows are
DESTINATION nodes, ``col_ind`` holds SOURCE nodes, every per-edge tensor is in CSR
position order.

What each function follows in the reference, and what pins it:

* ``gat_forward`` / ``gat_layer_dgl`` -- ``GATConv_dgl.forward``
  (layers/gatconv_layer.py:196-213) with the fused op's orientation
  (layers/gatconv_layer.py:48-57; operators/fused_gat.py:52-71).  Pinned by
  ``gat_forward_dense`` (``torch.softmax`` over a dense masked score matrix), by
  the closed-form cases in tests (self-loop-only graph gives out == in_feat, the
  graph of script/inference/gatconv_test.py:75-76; zero attention gives the
  neighbour mean == a row-normalised scipy SpMM), and by the C restatement in
  ``fgnn_oracle.c`` written independently with explicit loops.
* ``edgeconv_forward`` -- ``EdgeConv_reorg.forward`` (layers/edgeconv_layer.py:102-109)
  == fused op contract (operators/fused_edgeconv.py:18-29).  Pinned by brute-force
  python loops with a strict ``>`` update (first maximum wins).
* ``gmm_forward`` -- ``GMMConv_dgl.forward`` (layers/gmmconv_layer.py:130-149).
  Pinned by the special case inv_sigma == 0 (weights 1, plain scipy SpMM) and the C
  restatement.
* ``csr2csc`` -- what the reference scripts do on the host with scipy
  (script/train/train_gmmconv_our.py:80-93); pinned by scipy ``tocsc`` and by a
  brute-force python placement.  The reference's own GPU transpose is cuSPARSE
  ``cusparseCsr2cscEx2`` (CUDA 11.3, src/csr2csc/csr2csc.cu:10-23), third-party and
  absent here: parity with *that* routine is unpinned; the contract is the stable
  (ascending CSR position) transpose.
* ``gmm_layer_dgl`` -- the whole ``GMMConv_dgl.forward`` (layers/gmmconv_layer.py:130-149: fc,
  ``view(-1, K, out)``, Gaussian-weighted sum, ``.sum(1)``, residual, bias).  Pinned by K = 1,
  inv_sigma = 0 (a scipy SpMM of ``feat @ W.T``), by a hand-built 3-node case with residual and
  bias worked out with python loops and ``math.exp``, and by a check that the other (out, K)
  view order gives a different result.
* ``gat_abs_sums`` / ``gmm_abs_sums`` -- not reference functions: for every output of the two
  fused operators the sum of the ABSOLUTE values of its elementary summands (products of inputs,
  no cancellation inside), which is what an fp32 rounding-error bound of a cancellation sum
  scales with.  Pinned by construction checks in tests (equal to |output| when all inputs are
  non-negative; never below |output|).
* ``gat_reference_chunked`` -- the same GAT math with the analytic backward and the scales, written
  without any [E,H,F] tensor so that it runs at the full benchmark sizes.  Pinned in tests against
  ``gat_forward`` + autograd and ``gat_abs_sums`` on small graphs with chunk sizes that cut rows.
* small operators -- one-line gather/scatter identities
  (operators/edge_softmax.py:30-42, operators/u_add_v.py:19-29,
  operators/mhspmm.py:24-41, operators/spmm.py:25-66).

Gradients come from ``torch.autograd`` through these float64 forms.
"""
from __future__ import annotations

import numpy as np
import torch


# --------------------------------------------------------------------------- helpers
def row_of_edge(row_ptr: torch.Tensor) -> torch.Tensor:
    """Destination node of every CSR position (int64)."""
    rp = row_ptr.to(torch.int64)
    deg = rp[1:] - rp[:-1]
    return torch.repeat_interleave(torch.arange(deg.numel(), dtype=torch.int64, device=rp.device), deg)


def _segment_softmax(e: torch.Tensor, dst: torch.Tensor, n: int):
    """Softmax of e[E,H] over edges sharing a destination.  Returns (alpha, max, sum)."""
    h = e.shape[1]
    idx = dst.view(-1, 1).expand(-1, h)
    mx = torch.full((n, h), -float("inf"), dtype=e.dtype, device=e.device)
    mx = mx.scatter_reduce(0, idx, e, reduce="amax", include_self=True)
    ex = torch.exp(e - mx[dst])
    sm = torch.zeros((n, h), dtype=e.dtype, device=e.device).index_add_(0, dst, ex)
    return ex / sm[dst], mx, sm


# --------------------------------------------------------------------------- GAT
def gat_forward(attn_row, attn_col, row_ptr, col_ind, negative_slope, in_feat,
                return_edge=False):
    """out[i,h,:] = sum_p softmax_p(lrelu(attn_row[i,h] + attn_col[j_p,h])) * in_feat[j_p,h,:].

    Follows GATConv_dgl.forward (layers/gatconv_layer.py:204-210): u_add_v, LeakyReLU,
    edge_softmax by destination, u_mul_e + sum.  Rows without edges give zeros
    (src/fused_gat/fused_gat_SM.cu:193-286 convention).
    """
    n = attn_row.shape[0]
    dst = row_of_edge(row_ptr)
    src = col_ind.to(torch.int64)
    e = torch.nn.functional.leaky_relu(attn_row[dst] + attn_col[src], negative_slope)
    alpha, mx, sm = _segment_softmax(e, dst, n)
    msg = alpha.unsqueeze(-1) * in_feat[src]
    out = torch.zeros_like(in_feat).index_add_(0, dst, msg)
    if return_edge:
        return out, e, alpha, mx, sm
    return out


def gat_forward_dense(attn_row, attn_col, row_ptr, col_ind, negative_slope, in_feat):
    """Brute force for tiny, duplicate-free graphs: dense masked torch.softmax."""
    n, h = attn_row.shape
    dst = row_of_edge(row_ptr)
    src = col_ind.to(torch.int64)
    mask = torch.zeros(n, n, dtype=torch.bool)
    mask[dst, src] = True
    s = attn_row.view(n, 1, h) + attn_col.view(1, n, h)          # [dst, src, h]
    s = torch.nn.functional.leaky_relu(s, negative_slope)
    s = s.masked_fill(~mask.unsqueeze(-1), -float("inf"))
    a = torch.softmax(s, dim=1)
    a = torch.nan_to_num(a, nan=0.0)                               # empty rows
    return torch.einsum("ijh,jhf->ihf", a, in_feat)


def gat_layer_ours(W, attn_l, attn_r, row_ptr, col_ind, negative_slope, feat):
    """Dense part + fused op as the reference's GATConv (layers/gatconv_layer.py:48-57):
    attn_l weights the destination (row) side, attn_r the source (column) side."""
    hh, ff = attn_l.shape[1], attn_l.shape[2]
    h = torch.matmul(feat, W).view(-1, hh, ff)
    attn_row = (attn_l * h).sum(-1)
    attn_col = (attn_r * h).sum(-1)
    return gat_forward(attn_row, attn_col, row_ptr, col_ind, negative_slope, h)


def gat_layer_dgl(fc_weight, attn_l, attn_r, row_ptr, col_ind, negative_slope, feat):
    """GATConv_dgl.forward (layers/gatconv_layer.py:196-213) written with explicit
    src/dst gathers: el on the SOURCE, er on the DESTINATION.  With fc_weight = W.T,
    attn_l(dgl) = attn_r(ours), attn_r(dgl) = attn_l(ours) it equals gat_layer_ours."""
    hh, ff = attn_l.shape[1], attn_l.shape[2]
    n = feat.shape[0]
    ft = torch.nn.functional.linear(feat, fc_weight).view(-1, hh, ff)
    el = (ft * attn_l).sum(-1)
    er = (ft * attn_r).sum(-1)
    dst = row_of_edge(row_ptr)
    src = col_ind.to(torch.int64)
    e = torch.nn.functional.leaky_relu(el[src] + er[dst], negative_slope)
    a, _, _ = _segment_softmax(e, dst, n)
    return torch.zeros_like(ft).index_add_(0, dst, a.unsqueeze(-1) * ft[src])


def gat_abs_sums(attn_row, attn_col, row_ptr, col_ind, negative_slope, in_feat, grad_out):
    """Sum of |elementary summand| for every output of the fused GAT forward and backward (the scale
    of their fp32 rounding error).  With alpha the attention, d = lrelu'(e) and
    geA[p,h] = sum_f |g[i,h,f]| |x[j,h,f]|, wsA[i,h] = sum_p alpha geA:
      out           sum_p alpha |x_j|
      grad_feat     sum_i alpha |g_i|
      grad_attn_row sum_p alpha |d| (geA + wsA[i])      (terms of src/fused_gat/fused_gat_SM.cu:656-732)
      grad_attn_col the same terms summed per source."""
    n = attn_row.shape[0]
    dst = row_of_edge(row_ptr)
    src = col_ind.to(torch.int64)
    _, e, alpha, _, _ = gat_forward(attn_row, attn_col, row_ptr, col_ind, negative_slope, in_feat, return_edge=True)
    ax, ag = in_feat.abs(), grad_out.abs()
    s_out = torch.zeros_like(ax).index_add_(0, dst, alpha.unsqueeze(-1) * ax[src])
    s_gfeat = torch.zeros_like(ax).index_add_(0, src, alpha.unsqueeze(-1) * ag[dst])
    ge_a = (ag[dst] * ax[src]).sum(-1)
    ws_a = torch.zeros_like(attn_row).index_add_(0, dst, alpha * ge_a)
    d = torch.where(e > 0, torch.ones_like(e), torch.full_like(e, abs(negative_slope)))
    t_a = alpha * d * (ge_a + ws_a[dst])
    s_gar = torch.zeros_like(attn_row).index_add_(0, dst, t_a)
    s_gac = torch.zeros_like(attn_row).index_add_(0, src, t_a)
    return {"out": s_out, "grad_feat": s_gfeat, "grad_attn_row": s_gar, "grad_attn_col": s_gac}


def segment_sums(ptr, vals):
    """out[r] = sum of vals[ptr[r]:ptr[r+1]] along dim 0 of vals [E,H] (empty segments give 0), by differences of
    one running sum per column (taken along the contiguous dimension of the transposed array: fast at 10^8
    entries, where index_add_ of float64 serialises on its atomics)."""
    c = torch.cumsum(vals.t().contiguous(), 1)
    c = torch.cat([torch.zeros_like(c[:, :1]), c], 1)
    p = ptr.to(torch.int64)
    return (c[:, p[1:]] - c[:, p[:-1]]).t().contiguous()


def segment_weighted_rows(ptr, ids, weights, feat):
    """out[r,h,:] = sum_{p in [ptr[r], ptr[r+1])} weights[p,h] * feat[ids[p],h,:] in float64 without the [E,H,F]
    message tensor of gat_forward: per head one sparse-matrix product by the library routine
    (torch.sparse.mm on a CSR matrix holding the weights; duplicate entries of a row are separate terms).
    feat may be float32."""
    n_rows = ptr.numel() - 1
    out = torch.empty((n_rows,) + tuple(feat.shape[1:]), dtype=torch.float64, device=feat.device)
    crow, col = ptr.to(torch.int64), ids.to(torch.int64)
    for h in range(feat.shape[1]):
        a = torch.sparse_csr_tensor(crow, col, weights[:, h].contiguous(), size=(n_rows, feat.shape[0]))
        out[:, h, :] = torch.sparse.mm(a, feat[:, h, :].double().contiguous())
    return out


def edge_dots(dst, src, a, b, chunk=1 << 20, absolute=False):
    """[E,H]: <a[dst[p],h,:], b[src[p],h,:]> in float64 (of the absolute values when `absolute`), in chunks."""
    out = torch.empty((dst.numel(), a.shape[1]), dtype=torch.float64, device=a.device)
    for s0 in range(0, dst.numel(), chunk):
        sl = slice(s0, min(s0 + chunk, dst.numel()))
        u, v = a[dst[sl]].double(), b[src[sl]].double()
        out[sl] = (u.abs() * v.abs()).sum(-1) if absolute else (u * v).sum(-1)
    return out


def gat_reference_chunked(attn_row, attn_col, row_ptr, col_ind, col_ptr, row_ind, permute, negative_slope, in_feat, grad_out,
                          chunk=1 << 20, log=None):
    """The whole fused GAT forward and backward in float64 with explicit formulas instead of autograd, and the
    scales of gat_abs_sums next to them, without any [E,H,F] tensor (sparse-matrix products per head, per-edge dot
    products in chunks): usable on the 10^8-edge graphs (on whatever device the inputs live on; they may be float32).  Same math as gat_forward; the backward terms are
    ge = <g_i, x_j>, ws_i = sum_p alpha ge, g_score = alpha (ge - ws_i) lrelu'(e)
    (src/fused_gat/fused_gat_SM.cu:656-732).  Returns a dict of out, grad_feat, grad_attn_row, grad_attn_col,
    S_<name> for each, and A_grad_attn_row / A_grad_attn_col (see below)."""
    log = log or (lambda msg: None)
    ar, ac = attn_row.double(), attn_col.double()
    dst = row_of_edge(row_ptr)
    src = col_ind.to(torch.int64)
    pm = permute.to(torch.int64)
    raw = ar[dst] + ac[src]
    # LeakyReLU' jumps at 0: an fp32 evaluation may land on the other side when the exact pre-activation is within
    # its rounding of the operands (2 * 2^-24 * (|attn_row| + |attn_col|)).  Such edges are marked; what the jump can
    # change in the score gradients is returned as an allowance (A_grad_attn_*), zero everywhere else.
    amb = raw.abs() <= 2.0 * 2.0 ** -24 * (ar.abs()[dst] + ac.abs()[src])
    e = torch.nn.functional.leaky_relu(raw, negative_slope)
    del raw
    alpha, _, _ = _segment_softmax(e, dst, ar.shape[0])
    d = torch.where(e > 0, 1.0, abs(negative_slope))
    del e
    log("attention weights done")
    res = {"out": segment_weighted_rows(row_ptr, col_ind, alpha, in_feat)}
    log("out done")
    res["S_out"] = segment_weighted_rows(row_ptr, col_ind, alpha, in_feat.abs())
    a_csc = alpha[pm]
    res["grad_feat"] = segment_weighted_rows(col_ptr, row_ind, a_csc, grad_out)
    log("grad_feat done")
    res["S_grad_feat"] = segment_weighted_rows(col_ptr, row_ind, a_csc, grad_out.abs())
    del a_csc
    ge = edge_dots(dst, src, grad_out, in_feat, chunk)
    log("edge dot products done")
    ws = segment_sums(row_ptr, alpha * ge)
    gs = alpha * (ge - ws[dst]) * torch.where(d == 1.0, 1.0, negative_slope)
    jump = torch.where(amb, (alpha * (ge - ws[dst])).abs() * abs(1.0 - negative_slope), 0.0)
    res["A_grad_attn_row"] = segment_sums(row_ptr, jump)
    res["A_grad_attn_col"] = segment_sums(col_ptr, jump[pm])
    del ge, ws, jump, amb
    res["grad_attn_row"] = segment_sums(row_ptr, gs)
    res["grad_attn_col"] = segment_sums(col_ptr, gs[pm])
    del gs
    ge_a = edge_dots(dst, src, grad_out, in_feat, chunk, absolute=True)
    ws_a = segment_sums(row_ptr, alpha * ge_a)
    t_a = alpha * d * (ge_a + ws_a[dst])
    del ge_a, ws_a
    res["S_grad_attn_row"] = segment_sums(row_ptr, t_a)
    res["S_grad_attn_col"] = segment_sums(col_ptr, t_a[pm])
    return res


def gat_layer_abs_sums(W, attn_l, attn_r, row_ptr, col_ind, negative_slope, feat, grad_out):
    """gat_abs_sums carried through the dense part of the layer (gat_layer_ours): the projected features
    are themselves sums, so their scale |feat| @ |W| takes the place of |in_feat|, and the parameter
    gradients are the op-level scales pushed through |feat|, |W|, |attn|."""
    hh, ff = attn_l.shape[1], attn_l.shape[2]
    n = feat.shape[0]
    h = torch.matmul(feat, W).view(-1, hh, ff)
    s_h = torch.matmul(feat.abs(), W.abs()).view(-1, hh, ff)
    s = gat_abs_sums((attn_l * h).sum(-1), (attn_r * h).sum(-1), row_ptr, col_ind, negative_slope, s_h, grad_out)
    s_gh = s["grad_feat"] + s["grad_attn_row"].unsqueeze(-1) * attn_l.abs() + s["grad_attn_col"].unsqueeze(-1) * attn_r.abs()
    return {"out": s["out"], "grad_feat": s_gh.view(n, -1) @ W.abs().t(), "grad_W": feat.abs().t() @ s_gh.view(n, -1),
            "grad_attn_l": (s["grad_attn_row"].unsqueeze(-1) * s_h).sum(0, keepdim=True),
            "grad_attn_r": (s["grad_attn_col"].unsqueeze(-1) * s_h).sum(0, keepdim=True)}


# --------------------------------------------------------------------------- EdgeConv
def edgeconv_forward(k, src_ind, h_src, h_dst):
    """out[i,f] = max_p (h_dst[i,f] + h_src[src_ind[p],f]), p in [i*k,(i+1)*k); argmax is the
    SOURCE NODE ID at the FIRST maximal position (layers/edgeconv_layer.py:102-109;
    operators/fused_edgeconv.py:18-29).  Implemented as an explicit running strict-'>' scan
    over the k neighbours so the tie rule is stated, not inherited from a library."""
    n, f = h_dst.shape
    src = src_ind.to(torch.int64).view(n, k)
    best = h_dst + h_src[src[:, 0]]
    arg = src[:, 0].view(n, 1).expand(n, f).clone()
    for t in range(1, k):
        v = h_dst + h_src[src[:, t]]
        upd = v > best
        best = torch.where(upd, v, best)
        arg = torch.where(upd, src[:, t].view(n, 1).expand(n, f), arg)
    return best, arg.to(torch.int32)


def edgeconv_forward_autograd(k, src_ind, h_src, h_dst):
    """Differentiable form (gather + amax) whose autograd is the backward oracle.  torch.max
    over a dim routes the gradient to ONE index; it is only used where maxima are unique."""
    n, f = h_dst.shape
    src = src_ind.to(torch.int64).view(n, k)
    v = h_dst.unsqueeze(1) + h_src[src]            # [n,k,f]
    return v.max(dim=1).values


def edgeconv_backward(max_idx, grad_out, n_src):
    """grad_src = scatter_add(grad_out at argmax); grad_dst = grad_out
    (operators/fused_edgeconv.py:26-29)."""
    f = grad_out.shape[1]
    g = torch.zeros(n_src, f, dtype=grad_out.dtype)
    cols = torch.arange(f).view(1, f).expand_as(max_idx)
    g.index_put_((max_idx.to(torch.int64), cols), grad_out, accumulate=True)
    return g, grad_out


# --------------------------------------------------------------------------- GMMConv
def gaussian(pseudo, mu, inv_sigma):
    """w[p,k] = exp(-0.5 * sum_d ((pseudo[p,d]-mu[k,d]) * inv_sigma[k,d])^2)
    (layers/gmmconv_layer.py:136-139)."""
    e, dim = pseudo.shape
    kk = mu.shape[0]
    g = -0.5 * ((pseudo.view(e, 1, dim) - mu.view(1, kk, dim)) ** 2)
    g = g * (inv_sigma.view(1, kk, dim) ** 2)
    return torch.exp(g.sum(-1))


def gmm_forward(row_ptr, col_ind, node_feat, pseudo, mu, inv_sigma):
    """out[i,k,:] = sum_p w[p,k] * node_feat[j_p,k,:] (layers/gmmconv_layer.py:140-142;
    operators/fused_gmmconv.py:43-48).  pseudo is in CSR position order."""
    dst = row_of_edge(row_ptr)
    src = col_ind.to(torch.int64)
    w = gaussian(pseudo, mu, inv_sigma)
    msg = w.unsqueeze(-1) * node_feat[src]
    return torch.zeros_like(node_feat).index_add_(0, dst, msg)


def gmm_abs_sums(row_ptr, col_ind, node_feat, pseudo, mu, inv_sigma, grad_out):
    """Sum of |elementary summand| for every output of the fused GMMConv forward and backward
    (see gat_abs_sums).  With gwA[p,k] = sum_f |g[i,k,f]| |x[j,k,f]| and t = pseudo - mu:
      out sum_p w |x_j|;  grad_feat sum_i w |g_i|;  grad_pseudo[p,d] sum_k gwA w |t| s^2;
      grad_mu[k,d] sum_p gwA w |t| s^2;  grad_sigma[k,d] sum_p gwA w t^2 |s|."""
    dst = row_of_edge(row_ptr)
    src = col_ind.to(torch.int64)
    w = gaussian(pseudo, mu, inv_sigma)
    ax, ag = node_feat.abs(), grad_out.abs()
    s_out = torch.zeros_like(ax).index_add_(0, dst, w.unsqueeze(-1) * ax[src])
    s_gx = torch.zeros_like(ax).index_add_(0, src, w.unsqueeze(-1) * ag[dst])
    gw_a = ((ag[dst] * ax[src]).sum(-1) * w).unsqueeze(-1)                  # [E,K,1]
    t = (pseudo.unsqueeze(1) - mu.unsqueeze(0)).abs()                       # [E,K,dim]
    sg = inv_sigma.abs().unsqueeze(0)
    return {"out": s_out, "grad_feat": s_gx, "grad_pseudo": (gw_a * t * sg * sg).sum(1),
            "grad_mu": (gw_a * t * sg * sg).sum(0), "grad_sigma": (gw_a * t * t * sg).sum(0)}


def gmm_layer_dgl(fc_weight, mu, inv_sigma, bias, row_ptr, col_ind, feat, pseudo, res_weight=None):
    """GMMConv_dgl.forward (layers/gmmconv_layer.py:130-149)."""
    kk = mu.shape[0]
    h = torch.nn.functional.linear(feat, fc_weight)
    h = h.view(feat.shape[0], kk, -1)
    rst = gmm_forward(row_ptr, col_ind, h, pseudo, mu, inv_sigma).sum(1)
    if res_weight is not None:
        rst = rst + torch.nn.functional.linear(feat, res_weight)
    if bias is not None:
        rst = rst + bias
    return rst


def gmm_layer_abs_sums(fc_weight, mu, inv_sigma, bias, row_ptr, col_ind, feat, pseudo, res_weight, grad_out):
    """gmm_abs_sums carried through the dense part of gmm_layer_dgl (fc, sum over kernels, residual, bias)."""
    kk = mu.shape[0]
    n = feat.shape[0]
    af, ag = feat.abs(), grad_out.abs()
    s_h = (af @ fc_weight.abs().t()).view(n, kk, -1)
    s = gmm_abs_sums(row_ptr, col_ind, s_h, pseudo, mu, inv_sigma, ag.unsqueeze(1).expand(-1, kk, -1))
    out = s["out"].sum(1)
    gfeat = s["grad_feat"].reshape(n, -1) @ fc_weight.abs()
    res = {"grad_fc": s["grad_feat"].reshape(n, -1).t() @ af, "grad_pseudo": s["grad_pseudo"], "grad_mu": s["grad_mu"],
           "grad_sigma": s["grad_sigma"], "grad_bias": ag.sum(0)}
    if res_weight is not None:
        out = out + af @ res_weight.abs().t()
        gfeat = gfeat + ag @ res_weight.abs()
        res["grad_res"] = ag.t() @ af
    if bias is not None:
        out = out + bias.abs()
    res["out"] = out
    res["grad_feat"] = gfeat
    return res


def multilinear_abs_sums(fn, inputs, grad_out):
    """For an operator that is a sum of products of its float inputs with no other sign in it (SpMM,
    SDDMM, u_add_v, a scatter-add): the scales of the output and of every input gradient are the operator
    and its autograd evaluated on the absolute values.  Returns (S_out, [S_grad of every input])."""
    leaves = [t.detach().abs().clone().requires_grad_(True) for t in inputs]
    out = fn(*leaves)
    out.backward(grad_out.abs())
    return out.detach(), [t.grad for t in leaves]


# --------------------------------------------------------------------------- csr2csc
def csr2csc(row_ptr, col_ind, n_cols=None):
    """Stable transpose: entries of a column ordered by ascending CSR position.
    Returns (col_ptr[int32], row_ind[int32], permute[int32]) with permute[q] = CSR position
    of CSC entry q -- what script/train/train_gmmconv_our.py:80-93 builds with scipy."""
    rp = np.asarray(row_ptr, dtype=np.int64)
    ci = np.asarray(col_ind, dtype=np.int64)
    n = rp.shape[0] - 1
    nc = n if n_cols is None else n_cols
    perm = np.argsort(ci, kind="stable")
    rows = np.repeat(np.arange(n, dtype=np.int64), np.diff(rp))
    col_ptr = np.zeros(nc + 1, dtype=np.int64)
    np.add.at(col_ptr, ci + 1, 1)
    col_ptr = np.cumsum(col_ptr)
    return (col_ptr.astype(np.int32), rows[perm].astype(np.int32), perm.astype(np.int32))


def csr2csc_bruteforce(row_ptr, col_ind, n_cols=None):
    """Python-loop placement for tiny inputs (independent of argsort)."""
    n = len(row_ptr) - 1
    nc = n if n_cols is None else n_cols
    buckets = [[] for _ in range(nc)]
    for i in range(n):
        for p in range(int(row_ptr[i]), int(row_ptr[i + 1])):
            buckets[int(col_ind[p])].append((i, p))
    col_ptr, row_ind, perm = [0], [], []
    for c in range(nc):
        for (i, p) in buckets[c]:
            row_ind.append(i)
            perm.append(p)
        col_ptr.append(len(row_ind))
    return (np.array(col_ptr, np.int32), np.array(row_ind, np.int32), np.array(perm, np.int32))


# --------------------------------------------------------------------------- small operators
def edge_softmax(row_ptr, h):
    """Per-destination, per-head softmax of h[E,H] (operators/edge_softmax.py:30-42)."""
    n = row_ptr.shape[0] - 1
    a, _, _ = _segment_softmax(h, row_of_edge(row_ptr), n)
    return a


def u_add_v(row_ptr, col_ind, row_val, col_val):
    """out[p,:] = row_val[row(p),:] + col_val[col(p),:] (operators/u_add_v.py:19-29)."""
    return row_val[row_of_edge(row_ptr)] + col_val[col_ind.to(torch.int64)]


def mhspmm(row_ptr, col_ind, att, feat):
    """out[i,h,:] = sum_p att[p,h] * feat[j_p,h,:] (operators/mhspmm.py:24-41)."""
    dst = row_of_edge(row_ptr)
    msg = att.unsqueeze(-1) * feat[col_ind.to(torch.int64)]
    n_out = row_ptr.shape[0] - 1
    out = torch.zeros((n_out,) + tuple(feat.shape[1:]), dtype=feat.dtype)
    return out.index_add_(0, dst, msg)


def mhsddmm(row_ptr, col_ind, grad, feat):
    """out[p,h] = <grad[row(p),h,:], feat[col(p),h,:]> (src/sddmm/mhsddmm.cu:5-99)."""
    return (grad[row_of_edge(row_ptr)] * feat[col_ind.to(torch.int64)]).sum(-1)


def spmm(row_ptr, col_ind, x, csr_data=None):
    """out[i,:] = sum_p w[p] * x[j_p,:] with w == 1 when csr_data is None (operators/spmm.py:25-66)."""
    dst = row_of_edge(row_ptr)
    msg = x[col_ind.to(torch.int64)]
    if csr_data is not None:
        msg = msg * csr_data.view(-1, 1)
    n_out = row_ptr.shape[0] - 1
    return torch.zeros((n_out, x.shape[1]), dtype=x.dtype).index_add_(0, dst, msg)


def sddmm(row_ptr, col_ind, a, b):
    """out[p] = <a[row(p),:], b[col(p),:]> (src/sddmm/sddmm.cu:5-359, unscaled form)."""
    return (a[row_of_edge(row_ptr)] * b[col_ind.to(torch.int64)]).sum(-1)

"""GPU results against the committed golden fixtures (tests/golden/*.npz, written by
tests/golden/make_golden.py from the float64 oracle)."""
import os

import numpy as np
import pytest
import torch

from oracle import fgnn_oracle as orc
from tests.util import assert_close, assert_close_sum, c_exp

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _gat_check(d, got):
    """(out, grad_x, grad_attn_row, grad_attn_col) against the fixture; the bar of every output comes from the sum of
    its absolute summands (oracle.gat_abs_sums on the fixture's inputs)."""
    h = {k: torch.from_numpy(d[k]).double() for k in ("attn_row", "attn_col", "x", "grad_out")}
    s = orc.gat_abs_sums(h["attn_row"], h["attn_col"], torch.from_numpy(d["row_ptr"]), torch.from_numpy(d["col_ind"]), float(d["slope"]),
                         h["x"], h["grad_out"])
    c = c_exp(float(h["attn_row"].abs().max() + h["attn_col"].abs().max()))
    for val, key, sk in zip(got, ("out", "grad_x", "grad_attn_row", "grad_attn_col"), ("out", "grad_feat", "grad_attn_row", "grad_attn_col")):
        assert_close_sum(val, torch.from_numpy(d[key]), s[sk], key, c=c)


def _t(a, dtype=None):
    t = torch.from_numpy(np.asarray(a))
    return (t if dtype is None else t.to(dtype)).to(DEV)


@pytest.mark.parametrize("name", ["gat_rmat_h4f16.npz", "gat_uniform_h2f6.npz"])
@pytest.mark.parametrize("variant", ["sm", "stash"])
def test_gat_golden(name, variant):
    from ae_mlsys_gnn_amd.operators import fused_gat as fg
    d = np.load(os.path.join(HERE, name))
    x = _t(d["x"]).requires_grad_(True); ar = _t(d["attn_row"]).requires_grad_(True); ac = _t(d["attn_col"]).requires_grad_(True)
    rp, ci, cp, ri, pm = (_t(d[k]) for k in ("row_ptr", "col_ind", "col_ptr", "row_ind", "permute"))
    if variant == "sm":
        out = fg.fused_gat_op(ar, ac, rp, ci, cp, ri, float(d["slope"]), x)
    else:
        out = fg.fused_gat_stash_op(ar, ac, rp, ci, cp, ri, float(d["slope"]), x, pm)
    out.backward(_t(d["grad_out"]))
    _gat_check(d, (out, x.grad, ar.grad, ac.grad))


def test_gat_backward_without_saved_aux_recomputes():
    # the reference's gat_backward signature carries no out/out2/c: the library recomputes them
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    d = np.load(os.path.join(HERE, "gat_rmat_h4f16.npz"))
    x, ar, ac = _t(d["x"]), _t(d["attn_row"]), _t(d["attn_col"])
    rp, ci, cp, ri = (_t(d[k]) for k in ("row_ptr", "col_ind", "col_ptr", "row_ind"))
    out, emax, esum, _, _, _, _ = gat_native.gat_forward(ar, ac, rp, ci, float(d["slope"]), x, need_aux=False)
    gx, gar, gac = gat_native.gat_backward(float(d["slope"]), rp, ci, cp, ri, emax, esum, x, ar, ac, _t(d["grad_out"]))
    _gat_check(d, (out, gx, gar, gac))


def test_gat_is_bit_reproducible():
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    d = np.load(os.path.join(HERE, "gat_rmat_h4f16.npz"))
    x, ar, ac, go = _t(d["x"]), _t(d["attn_row"]), _t(d["attn_col"]), _t(d["grad_out"])
    rp, ci, cp, ri = (_t(d[k]) for k in ("row_ptr", "col_ind", "col_ptr", "row_ind"))
    runs = []
    for _ in range(3):
        o = gat_native.gat_forward(ar, ac, rp, ci, 0.2, x)
        g = gat_native.gat_backward(0.2, rp, ci, cp, ri, o[1], o[2], x, ar, ac, go, out_feat=o[0], out2=o[3], cc=o[4])
        runs.append((o[0], *g))
    for r in runs[1:]:
        assert all(torch.equal(a, b) for a, b in zip(r, runs[0]))


def test_edgeconv_golden_bit_exact():
    from ae_mlsys_gnn_amd.operators.fused_edgeconv import edgeconv_native
    d = np.load(os.path.join(HERE, "edgeconv_k20_f64.npz"))
    out, arg = edgeconv_native.edgeconv_forward(int(d["k"]), _t(d["src_ind"]), _t(d["h_src"]), _t(d["h_dst"]))
    assert np.array_equal(arg.cpu().numpy(), d["argmax"])
    assert np.array_equal(out.cpu().numpy(), d["out"])


def test_gmm_golden():
    from ae_mlsys_gnn_amd.operators import fused_gmmconv as fg
    d = np.load(os.path.join(HERE, "gmm_k3_d2_f16.npz"))
    leaves = [_t(d[k]).requires_grad_(True) for k in ("x", "pseudo", "mu", "inv_sigma")]
    rp, ci, cp, ri, pm = (_t(d[k]) for k in ("row_ptr", "col_ind", "col_ptr", "row_ind", "permute"))
    out = fg.GmmConvFuse(rp, ci, cp, ri, pm, *leaves)
    out.backward(_t(d["grad_out"]))
    h = [torch.from_numpy(d[k]).double() for k in ("x", "pseudo", "mu", "inv_sigma", "grad_out")]
    s = orc.gmm_abs_sums(torch.from_numpy(d["row_ptr"]), torch.from_numpy(d["col_ind"]), *h)
    c = c_exp(float((0.5 * (((h[1].unsqueeze(1) - h[2].unsqueeze(0)) * h[3].unsqueeze(0)) ** 2).sum(-1)).max()))
    for val, key, sk in zip((out,) + tuple(t.grad for t in leaves), ("out", "grad_x", "grad_pseudo", "grad_mu", "grad_sigma"),
                            ("out", "grad_feat", "grad_pseudo", "grad_mu", "grad_sigma")):
        assert_close_sum(val, torch.from_numpy(d[key]), s[sk], key, c=c)


def test_csr2csc_golden_bit_exact():
    from ae_mlsys_gnn_amd.operators import csr2csc as op
    for name in ("gat_rmat_h4f16.npz", "gmm_k3_d2_f16.npz", "gat_uniform_h2f6.npz"):
        d = np.load(os.path.join(HERE, name))
        cp, ri, pm = op.csr2csc(_t(d["row_ptr"]), _t(d["col_ind"]))
        assert np.array_equal(cp.cpu().numpy(), d["col_ptr"])
        assert np.array_equal(ri.cpu().numpy(), d["row_ind"])
        assert np.array_equal(pm.cpu().numpy(), d["permute"])

"""GPU results against the committed golden fixtures (tests/golden/*.npz, written by
tests/golden/make_golden.py from the float64 oracle)."""
import os

import numpy as np
import pytest
import torch

from tests.util import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


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
    assert_close(out, torch.from_numpy(d["out"]), "out")
    assert_close(x.grad, torch.from_numpy(d["grad_x"]), "grad_x")
    assert_close(ar.grad, torch.from_numpy(d["grad_attn_row"]), "grad_attn_row", atol=1e-4)
    assert_close(ac.grad, torch.from_numpy(d["grad_attn_col"]), "grad_attn_col", atol=1e-4)


def test_gat_backward_without_saved_aux_recomputes():
    # the reference's gat_backward signature carries no out/out2/c: the library recomputes them
    from ae_mlsys_gnn_amd.operators.fused_gat import gat_native
    d = np.load(os.path.join(HERE, "gat_rmat_h4f16.npz"))
    x, ar, ac = _t(d["x"]), _t(d["attn_row"]), _t(d["attn_col"])
    rp, ci, cp, ri = (_t(d[k]) for k in ("row_ptr", "col_ind", "col_ptr", "row_ind"))
    out, emax, esum, _, _, _, _ = gat_native.gat_forward(ar, ac, rp, ci, float(d["slope"]), x, need_aux=False)
    gx, gar, gac = gat_native.gat_backward(float(d["slope"]), rp, ci, cp, ri, emax, esum, x, ar, ac, _t(d["grad_out"]))
    assert_close(out, torch.from_numpy(d["out"]), "out")
    assert_close(gx, torch.from_numpy(d["grad_x"]), "grad_x")
    assert_close(gar, torch.from_numpy(d["grad_attn_row"]), "grad_attn_row", atol=1e-4)
    assert_close(gac, torch.from_numpy(d["grad_attn_col"]), "grad_attn_col", atol=1e-4)


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
    assert_close(out, torch.from_numpy(d["out"]), "out")
    assert_close(leaves[0].grad, torch.from_numpy(d["grad_x"]), "grad_x")
    assert_close(leaves[1].grad, torch.from_numpy(d["grad_pseudo"]), "grad_pseudo", atol=1e-4)
    assert_close(leaves[2].grad, torch.from_numpy(d["grad_mu"]), "grad_mu", rtol=1e-3, atol=1e-2)
    assert_close(leaves[3].grad, torch.from_numpy(d["grad_sigma"]), "grad_sigma", rtol=1e-3, atol=1e-2)


def test_csr2csc_golden_bit_exact():
    from ae_mlsys_gnn_amd.operators import csr2csc as op
    for name in ("gat_rmat_h4f16.npz", "gmm_k3_d2_f16.npz", "gat_uniform_h2f6.npz"):
        d = np.load(os.path.join(HERE, name))
        cp, ri, pm = op.csr2csc(_t(d["row_ptr"]), _t(d["col_ind"]))
        assert np.array_equal(cp.cpu().numpy(), d["col_ptr"])
        assert np.array_equal(ri.cpu().numpy(), d["row_ind"])
        assert np.array_equal(pm.cpu().numpy(), d["permute"])

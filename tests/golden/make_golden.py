"""Writes the golden fixtures of this directory from seeded inputs and the float64 CPU oracle.

The reference ships no test vectors for this path and cannot be imported here (it JIT-compiles
CUDA sources at import), so the fixtures hold the oracle's outputs; the oracle itself is pinned
in tests/test_oracle.py against dense brute force, closed forms, scipy and an independent C
restatement.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from ae_mlsys_gnn_amd import graphs  # noqa: E402
from oracle import fgnn_oracle as orc  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def gat_case(name, g, h, f, slope, seed):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(g.n, h, f, generator=gen).double().requires_grad_(True)
    ar = torch.randn(g.n, h, generator=gen).double().requires_grad_(True)
    ac = torch.randn(g.n, h, generator=gen).double().requires_grad_(True)
    go = torch.randn(g.n, h, f, generator=gen).double()
    out = orc.gat_forward(ar, ac, g.row_ptr, g.col_ind, slope, x)
    out.backward(go)
    cp, ri, pm = orc.csr2csc(g.row_ptr.numpy(), g.col_ind.numpy())
    np.savez_compressed(os.path.join(HERE, name), row_ptr=g.row_ptr.numpy(), col_ind=g.col_ind.numpy(), col_ptr=cp, row_ind=ri,
                        permute=pm, slope=np.float64(slope), x=x.detach().numpy().astype(np.float32),
                        attn_row=ar.detach().numpy().astype(np.float32), attn_col=ac.detach().numpy().astype(np.float32),
                        grad_out=go.numpy().astype(np.float32), out=out.detach().numpy(), grad_x=x.grad.numpy(),
                        grad_attn_row=ar.grad.numpy(), grad_attn_col=ac.grad.numpy())


def edgeconv_case(name, bsz, npts, k, f, seed):
    gen = torch.Generator().manual_seed(seed)
    pts = torch.rand(bsz, npts, 3, generator=gen) * 2 - 1
    src = graphs.knn_graph(pts, k)
    hs = torch.round(torch.randn(bsz * npts, f, generator=gen) * 4) / 4     # coarse grid: exact ties occur
    hd = torch.round(torch.randn(bsz * npts, f, generator=gen) * 4) / 4
    out, arg = orc.edgeconv_forward(k, src, hs, hd)
    np.savez_compressed(os.path.join(HERE, name), k=np.int32(k), src_ind=src.numpy(), h_src=hs.numpy(), h_dst=hd.numpy(),
                        out=out.numpy(), argmax=arg.numpy())


def gmm_case(name, g, k, dim, f, seed):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(g.n, k, f, generator=gen).double().requires_grad_(True)
    ps = torch.rand(g.n_edges, dim, generator=gen).double().requires_grad_(True)
    mu = torch.rand(k, dim, generator=gen).double().requires_grad_(True)
    sg = (0.5 + torch.rand(k, dim, generator=gen)).double().requires_grad_(True)
    go = torch.randn(g.n, k, f, generator=gen).double()
    out = orc.gmm_forward(g.row_ptr, g.col_ind, x, ps, mu, sg)
    out.backward(go)
    cp, ri, pm = orc.csr2csc(g.row_ptr.numpy(), g.col_ind.numpy())
    np.savez_compressed(os.path.join(HERE, name), row_ptr=g.row_ptr.numpy(), col_ind=g.col_ind.numpy(), col_ptr=cp, row_ind=ri,
                        permute=pm, x=x.detach().numpy().astype(np.float32), pseudo=ps.detach().numpy().astype(np.float32),
                        mu=mu.detach().numpy().astype(np.float32), inv_sigma=sg.detach().numpy().astype(np.float32),
                        grad_out=go.numpy().astype(np.float32), out=out.detach().numpy(), grad_x=x.grad.numpy(),
                        grad_pseudo=ps.grad.numpy(), grad_mu=mu.grad.numpy(), grad_sigma=sg.grad.numpy())


if __name__ == "__main__":
    gat_case("gat_rmat_h4f16.npz", graphs.rmat_graph(300, 4000, seed=1), 4, 16, 0.2, 11)
    gat_case("gat_uniform_h2f6.npz", graphs.uniform_graph(200, 1500, seed=2), 2, 6, 0.05, 12)
    edgeconv_case("edgeconv_k20_f64.npz", 2, 128, 20, 64, 13)
    gmm_case("gmm_k3_d2_f16.npz", graphs.rmat_graph(250, 3000, seed=3), 3, 2, 16, 14)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))

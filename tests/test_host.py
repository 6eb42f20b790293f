"""CPU-side checks of the host logic: the C ABI library loads and exports every declared symbol,
operators refuse to run without a GPU (no silent CPU fallback), graph builders are well formed."""
import ctypes
import os
import re

import pytest
import torch

from ae_mlsys_gnn_amd import _lib, graphs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    txt = open(os.path.join(ROOT, "include", "fgnn.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(fgnn_[a-z0-9_]+)\s*\(", txt)))


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_lib.LIB_PATH), "libfgnn_hip.so has not been built (python -m ae_mlsys_gnn_amd.build)"
    names = _header_symbols()
    assert len(names) >= 29
    handle = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, "declared in include/fgnn.h but not exported: %s" % missing
    assert names == _lib.exported_symbols(), "ctypes signature table out of step with include/fgnn.h"
    assert _lib.lib().fgnn_version() >= 100


def test_only_the_c_abi_is_exported():
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True).stdout
    funcs = [l.split()[-1] for l in out.splitlines() if " T " in l]
    assert funcs and all(f.startswith("fgnn_") for f in funcs), [f for f in funcs if not f.startswith("fgnn_")]


def test_operators_refuse_cpu_tensors():
    from ae_mlsys_gnn_amd.operators import fused_gat, fused_edgeconv, fused_gmmconv
    g = graphs.add_csc_torch(graphs.uniform_graph(16, 40))
    x = torch.randn(16, 2, 4); a = torch.randn(16, 2)
    with pytest.raises(_lib.FgnnError):
        fused_gat.fused_gat_op(a, a, g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, 0.2, x)
    with pytest.raises(_lib.FgnnError):
        fused_edgeconv.fused_edgeconv_op(2, torch.zeros(32, dtype=torch.int32), torch.randn(16, 4), torch.randn(16, 4))
    with pytest.raises(_lib.FgnnError):
        fused_gmmconv.GaussianCp(torch.rand(5, 2), torch.rand(3, 2), torch.rand(3, 2))


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(ROOT, "does_not_exist.so"))
    with pytest.raises(_lib.FgnnError, match="missing"):
        _lib.lib()


def test_argument_errors_without_gpu():
    # argument validation happens before any launch, so the error codes are observable on a CPU box
    l = _lib.lib()
    assert l.fgnn_gat_forward(4, 4, 1, 4, None, None, None, None, 0.2, None, None, None, None, None, None, None, None, None, None, 0, None) == -1
    assert b"NULL" in l.fgnn_last_error()
    assert l.fgnn_edgeconv_forward(4, 4, 0, 2, None, None, None, None, None, None) == -2
    assert l.fgnn_mhsddmm(4, 4, 65, 4, None, None, None, None, None, None) == -4
    assert l.fgnn_csr2csc(-1, 4, 4, None, None, None, None, None, None, 0, None) == -2
    assert l.fgnn_schedule_num_items(None) == 0


def test_graph_builders():
    g = graphs.rmat_graph(500, 6000, seed=1)
    rp, ci = g.row_ptr.long(), g.col_ind.long()
    assert rp[0] == 0 and rp[-1] == g.n_edges and bool((rp[1:] >= rp[:-1]).all())
    dst = torch.repeat_interleave(torch.arange(g.n), rp[1:] - rp[:-1])
    keys = dst * g.n + ci
    assert bool((keys[1:] > keys[:-1]).all()), "edges must be unique and sorted by (dst, src)"
    assert int((dst == ci).sum()) == g.n, "exactly one self loop per node"
    assert g.n_edges == 6000 + g.n
    g2 = graphs.rmat_graph(500, 6000, seed=1)
    assert torch.equal(g.col_ind, g2.col_ind)
    deg = rp[1:] - rp[:-1]
    assert int(deg.max()) > 4 * float(deg.float().mean()), "R-MAT should be heavy tailed"
    pts = torch.rand(3, 50, 3)
    src = graphs.knn_graph(pts, 7).view(3, 50, 7)
    assert bool((src[:, :, 0] == torch.arange(150).view(3, 50)).all()), "nearest neighbour of a point is itself"
    assert bool(((src // 50) == torch.arange(3).view(3, 1, 1)).all()), "neighbours stay inside the cloud"

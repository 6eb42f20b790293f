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
    # the same graph with its node labels permuted: a valid sorted CSR, the same in- and out-degree multisets, one self loop
    # per node, reproducible by seed, and the hubs no longer at the generator's ids
    gp = graphs.rmat_graph(500, 6000, seed=1, permute_labels=True)
    rpp, cip = gp.row_ptr.long(), gp.col_ind.long()
    dstp = torch.repeat_interleave(torch.arange(gp.n), rpp[1:] - rpp[:-1])
    kp = dstp * gp.n + cip
    assert gp.n_edges == g.n_edges and bool((kp[1:] > kp[:-1]).all()) and int((dstp == cip).sum()) == gp.n
    assert torch.equal(torch.sort(rpp[1:] - rpp[:-1]).values, torch.sort(deg).values)
    assert torch.equal(torch.sort(torch.bincount(cip, minlength=gp.n)).values, torch.sort(torch.bincount(ci, minlength=g.n)).values)
    assert torch.equal(gp.col_ind, graphs.rmat_graph(500, 6000, seed=1, permute_labels=True).col_ind)
    assert not torch.equal(rpp, rp)
    pts = torch.rand(3, 50, 3)
    src = graphs.knn_graph(pts, 7).view(3, 50, 7)
    assert bool((src[:, :, 0] == torch.arange(150).view(3, 50)).all()), "nearest neighbour of a point is itself"
    assert bool(((src // 50) == torch.arange(3).view(3, 1, 1)).all()), "neighbours stay inside the cloud"


def test_reference_import_recipe_resolves_to_this_package(tmp_path, monkeypatch):
    """The aliasing recipe documented for the reference tree: `operators` resolves to this package's
    mirror, so a layer file written against the reference's module names imports unchanged."""
    import importlib
    import sys
    import ae_mlsys_gnn_amd.operators as ops
    for name in ("operators", "operators.fused_gat", "operators.fused_edgeconv", "operators.fused_gmmconv", "operators.mhspmm",
                 "operators.edge_softmax", "operators.u_add_v", "operators.spmm", "operators.csr2csc"):
        monkeypatch.delitem(sys.modules, name, raising=False)
    monkeypatch.setitem(sys.modules, "operators", ops)
    for m in ("fused_gat", "fused_edgeconv", "fused_gmmconv", "mhspmm", "edge_softmax", "u_add_v", "spmm", "csr2csc"):
        monkeypatch.setitem(sys.modules, "operators." + m, getattr(ops, m))
    # a stand-in layer file using the reference's import lines (layers/gatconv_layer.py:7, edgeconv_layer.py:4,
    # gmmconv_layer.py:9-12)
    (tmp_path / "ref_style_layer.py").write_text(
        "from operators.fused_gat import fused_gat_op, fused_gat_stash_op, fused_gat_fusescatter\n"
        "from operators.fused_edgeconv import fused_edgeconv_op\n"
        "from operators.fused_gmmconv import GmmConvFuse, GmmConvStash, GaussianCp\n"
        "from operators.mhspmm import csrmhspmm\n"
        "from operators.edge_softmax import csr_edge_softmax\n"
        "from operators.u_add_v import u_add_v_op\n"
        "from operators.spmm import csrspmm\n"
        "from operators.csr2csc import sparsetrans\n")
    monkeypatch.syspath_prepend(str(tmp_path))
    mod = importlib.import_module("ref_style_layer")
    assert mod.fused_gat_op is ops.fused_gat.fused_gat_op and mod.sparsetrans is ops.csr2csc.sparsetrans


def test_reference_signatures_are_kept():
    """The public callables take the reference's arguments, by the same names and in the same order
    (operators/*.py, layers/*.py); anything this build adds comes after them and is optional."""
    import inspect
    from ae_mlsys_gnn_amd import layers, operators as ops
    want = {
        ops.fused_gat.fused_gat_op: "attn_row attn_col row_ptr col_ind col_ptr row_ind negative_slope in_feat save_memory",
        ops.fused_gat.fused_gat_stash_op: "attn_row attn_col row_ptr col_ind col_ptr row_ind negative_slope in_feat permute",
        ops.fused_gat.fused_gat_fusescatter: "attn_row attn_col row_ptr col_ind col_ptr row_ind negative_slope in_feat permute",
        ops.fused_edgeconv.fused_edgeconv_op: "k src_ind h_src h_dst",
        ops.fused_gmmconv.GmmConvFuse: "rowptr colind colptr rowind permute node_feat pseudo mu sigma",
        ops.fused_gmmconv.GmmConvStash: "rowptr colind colptr rowind permute node_feat pseudo mu sigma",
        ops.fused_gmmconv.GmmConvFuseEb: "rowptr colind colptr rowind permute node_feat pseudo mu sigma",
        ops.fused_gmmconv.GaussianCp: "pseudo mu sigma",
        ops.mhspmm.csrmhspmm: "rowptr colind colptr rowind permute feat attention",
        ops.edge_softmax.csr_edge_softmax: "rowptr h",
        ops.u_add_v.u_add_v_op: "row_ptr col_ind row_val col_val",
        ops.spmm.csrspmm: "rowptr colind x csr_data sym actnn",
        ops.csr2csc.sparsetrans: "rowptr colind numlist",
        layers.GATConv.forward: "self row_ptr col_ind col_ptr row_ind feat save_memory",
        layers.GATConv_stash.forward: "self row_ptr col_ind col_ptr row_ind feat permute",
        layers.EdgeConv.forward: "self k src_ind feat",
        layers.GMMConv.forward: "self rowptr colind colptr rowind permute feat pseudo",
        layers.GATConv.__init__: "self in_feats out_feats num_heads negative_slope",
        layers.EdgeConv.__init__: "self in_feat out_feat batch_norm allow_zero_in_degree",
        layers.GMMConv.__init__: "self in_feats out_feats dim n_kernels aggregator_type residual bias allow_zero_in_degree",
    }
    for fn, names in want.items():
        params = inspect.signature(fn).parameters
        ref = names.split()
        assert list(params)[:len(ref)] == ref, fn
        assert all(params[extra].default is not inspect.Parameter.empty for extra in list(params)[len(ref):]), fn


def test_more_argument_errors_without_gpu():
    l = _lib.lib()
    assert l.fgnn_knn_graph(1, 10, 3, 11, None, None, None) == -2                 # k > P
    assert l.fgnn_gather_rows(5, 0, None, None, None, None) == -2                 # W < 1
    assert l.fgnn_edge_softmax(-1, 0, 1, None, None, None, None) == -2
    assert l.fgnn_gaussian(4, 1, 2, None, None, None, None, None) == -1
    assert l.fgnn_coo2csr(4, 4, 3, None, None, 1, None, None, None, None, None, 0, None) == -1
    out = ctypes.c_void_p()
    assert l.fgnn_schedule_create(None, 4, 0, None, ctypes.byref(out)) == -1
    assert l.fgnn_schedule_create_bucketed(None, None, 4, 0, 0, 1, None, ctypes.byref(out)) == -1
    l.fgnn_schedule_destroy(None)                                                  # no-op on NULL


def test_xcd_mapping_rule_without_gpu():
    """The rule behind the XCD-aware work lists: only a gfx950 device that shows all 256 compute units (eight XCDs of 32)
    is known to spread workgroups round-robin over eight XCDs; a partition of the part or another part gets plain lists."""
    l = _lib.lib()
    assert l.fgnn_xcd_mapping_for(b"gfx950:sramecc+:xnack-", 256) == 8
    assert l.fgnn_xcd_mapping_for(b"gfx950", 256) == 8
    assert l.fgnn_xcd_mapping_for(b"gfx950:sramecc+:xnack-", 128) == 0      # DPX: two devices of four XCDs
    assert l.fgnn_xcd_mapping_for(b"gfx950:sramecc+:xnack-", 32) == 0       # CPX: one XCD per device
    assert l.fgnn_xcd_mapping_for(b"gfx942:sramecc+:xnack-", 304) == 0
    assert l.fgnn_xcd_mapping_for(b"gfx9500", 256) == 0
    assert l.fgnn_xcd_mapping_for(None, 256) == 0
    assert l.fgnn_schedule_num_buckets(None) == 0


def test_column_sum_and_wide_row_argument_errors_without_gpu():
    l = _lib.lib()
    out = ctypes.c_void_p()
    assert l.fgnn_colsum_plan_create(None, None, 4, 4, 3, 8, 0, 0, None, ctypes.byref(out)) == -1
    assert l.fgnn_colsum_plan_create(None, None, 4, 4, 0, 8, 0, 0, None, None) == -1
    assert l.fgnn_edge_colsum(None, 8, None, None, None, 0, None) == -1
    assert l.fgnn_colsum_workspace_bytes(None, 8) == 0 and l.fgnn_colsum_plan_device_bytes(None) == 0
    l.fgnn_colsum_plan_destroy(None)
    assert l.fgnn_edge_rowsum(-1, 0, 8, None, None, None, None) == -2
    assert l.fgnn_u_add_v_backward_planned(4, 3, 8, None, None, None, None, None, None, None, 0, None) == -1
    # more than 1024 floats per head is the one width the GAT entries refuse; rows of many heads are grouped
    assert l.fgnn_gat_forward(4, 3, 2, 1028, None, None, None, None, 0.2, None, None, None, None, None, None, None, None, None, None, 0, None) == -4
    assert b"1024" in l.fgnn_last_error()
    assert l.fgnn_gat_forward(4, 3, 65, 4, None, None, None, None, 0.2, None, None, None, None, None, None, None, None, None, None, 0, None) == -4
    assert l.fgnn_mhsddmm(4, 3, 2, 1028, None, None, None, None, None, None) == -4
    # the workspace of a wide-row backward counts the head-group slices (and the stash slice when bit 1 is set)
    narrow = l.fgnn_gat_backward_workspace_bytes(1000, 4, 256, None, None, 0)
    wide = l.fgnn_gat_backward_workspace_bytes(1000, 8, 256, None, None, 0)
    assert wide > narrow + 5 * 1000 * 1024 * 4

"""The work lists (schedules) built on the device against the host-side builder they replace: item for item and
split for split the same list, for plain and XCD-aware lists, over segment lengths, bucket cut-offs and graph shapes
(empty rows, hubs, no edges at all, a single row); malformed pointer arrays are refused by both before any kernel
walks the index array with them."""
import pytest
import torch

from tests.util import custom_graph, degree_edge_graph
from ae_mlsys_gnn_amd import graphs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(monkeypatch, ptr, idx, seg_len, min_deg, with_positions=True):
    from ae_mlsys_gnn_amd import _lib
    out = []
    for builder in ("device", "host"):
        monkeypatch.setenv("FGNN_SCHEDULE_BUILDER", builder)
        s = _lib.Schedule(ptr, seg_len, idx, min_deg, with_positions=with_positions)
        items, splits = s.export()
        pos = s.take_positions() if (idx is not None and with_positions) else None
        out.append((s.n_items, s.n_partials, s.n_edges, items.cpu(), splits.cpu(), None if pos is None else pos.cpu(), s.device_bytes(),
                    s.n_wave_slots, s.n_buckets))
    monkeypatch.delenv("FGNN_SCHEDULE_BUILDER")
    return out


GRAPHS = {
    "degrees": lambda: degree_edge_graph(n=700, seed=0),
    "rmat": lambda: graphs.rmat_graph(3000, 200000, seed=8),
    "uniform": lambda: graphs.uniform_graph(2000, 30000, seed=2),
    "no_edges": lambda: custom_graph([[], [], [], [], []]),
    "one_row": lambda: custom_graph([list(range(1)) * 700]),
    "hub_only": lambda: custom_graph([[0] * 5000, [], [1]]),
}


@pytest.mark.parametrize("name", sorted(GRAPHS))
@pytest.mark.parametrize("seg_len,min_deg", [(0, 0), (64, 16), (128, 16), (256, 64), (192, 100), (2048, 1)])
def test_device_built_schedules_equal_the_host_built_ones(name, seg_len, min_deg, monkeypatch):
    g = GRAPHS[name]().to(DEV)
    for idx in (None, g.col_ind):
        dev, host = _both(monkeypatch, g.row_ptr, idx, seg_len, min_deg)
        assert dev[:3] == host[:3], (name, "bucketed" if idx is not None else "plain", dev[:3], host[:3])
        assert torch.equal(dev[3], host[3]), "work items differ"
        assert torch.equal(dev[4], host[4]), "split tables differ"
        if idx is not None:
            assert torch.equal(dev[5], host[5]), "position maps differ"
        assert dev[6] == host[6]
        # the long items are a prefix of the list: nothing longer than 64 entries from slot n_wave_slots on, and the mark
        # is tight to the 64 slots (per source bucket) it is rounded up to
        for n_wave, n_buckets, items in ((dev[7], dev[8], dev[3]), (host[7], host[8], host[3])):
            length = (items[:, 2] - items[:, 1]) * (items[:, 0] >= 0)
            per = 64 * max(n_buckets, 1)
            assert 0 <= n_wave <= len(items) and (n_wave % per == 0 or n_wave == len(items))
            assert n_wave == len(items) or int(length[n_wave:].max()) <= 64
            if n_wave > 0:
                assert int(length[max(n_wave - per, 0):n_wave].max()) > 64 or n_wave == len(items)
            else:
                assert len(items) == 0 or int(length.max()) <= 64
        assert dev[7] == host[7]
        # the list covers every entry exactly once
        it = dev[3][dev[3][:, 0] >= 0].long()
        assert int((it[:, 2] - it[:, 1]).sum()) == g.n_edges


def test_malformed_pointer_arrays_are_refused_by_both_builders(monkeypatch):
    from ae_mlsys_gnn_amd import _lib
    g = graphs.rmat_graph(500, 20000, seed=3).to(DEV)
    dec = g.row_ptr.clone(); dec[100] = dec[101] + 5
    first = g.row_ptr.clone(); first[0] = 1
    for builder in ("device", "host"):
        monkeypatch.setenv("FGNN_SCHEDULE_BUILDER", builder)
        for bad, msg in ((dec, "decreases"), (first, r"ptr\[0\]")):
            for idx in (None, g.col_ind):
                with pytest.raises(_lib.FgnnError, match=msg):
                    _lib.Schedule(bad, 0, idx, 16)


@pytest.mark.parametrize("name", sorted(GRAPHS))
def test_row_length_statistics(name):
    """The two numbers behind the choice of the work list (entries held by rows longer than the limit, the longest row)
    against torch reductions on the host."""
    import ctypes
    from ae_mlsys_gnn_amd import _lib
    g = GRAPHS[name]()
    deg = (g.row_ptr[1:] - g.row_ptr[:-1]).long()
    ptr_dev = g.row_ptr.to(DEV)
    for limit in (0, 1, 64, 512):
        stats = (ctypes.c_int64 * 2)()
        _lib.check(_lib.lib().fgnn_row_length_stats(_lib.ptr(ptr_dev), g.n, limit, ctypes.cast(stats, ctypes.c_void_p), _lib.stream_ptr()),
                   "fgnn_row_length_stats")
        assert int(stats[0]) == int(deg[deg > limit].sum()) and int(stats[1]) == int(deg.max() if g.n else 0)


def test_scheduled_sddmm_refuses_lists_it_cannot_use(monkeypatch):
    """fgnn_mhsddmm_scheduled stores its results at the caller's positions: a list of another graph and a list built
    without the position map are refused before any kernel runs; a list whose map was handed out stores in its own
    entry order."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd._lib import lib, ptr, stream_ptr
    g = graphs.add_csc_torch(graphs.rmat_graph(500, 20000, seed=1)).to(DEV)
    other = graphs.rmat_graph(500, 20000, seed=2).to(DEV)
    n, h, f = g.n, 2, 8
    a = torch.randn(n, h, f, device=DEV)
    out = torch.empty(g.n_edges, h, device=DEV)

    def call(sched, graph=g):
        return lib().fgnn_mhsddmm_scheduled(n, graph.n_edges, h, f, ptr(graph.row_ptr), ptr(graph.col_ind), ptr(a), ptr(a), ptr(out), sched.handle,
                                            stream_ptr())
    good = _lib.Schedule(g.row_ptr, 0, g.col_ind, 16, with_positions=True)
    assert call(good) == 0
    plain = torch.empty_like(out)
    _lib.check(lib().fgnn_mhsddmm(n, g.n_edges, h, f, ptr(g.row_ptr), ptr(g.col_ind), ptr(a), ptr(a), ptr(plain), stream_ptr()), "fgnn_mhsddmm")
    assert torch.equal(out, plain)
    assert call(_lib.Schedule(other.row_ptr, 0, other.col_ind, 16, with_positions=True)) == -6
    assert b"another pointer array" in lib().fgnn_last_error()
    assert call(_lib.Schedule(g.row_ptr, 0, g.col_ind, 16, with_positions=False)) == -6
    assert b"edge positions" in lib().fgnn_last_error()
    taken = _lib.Schedule(g.row_ptr, 0, g.col_ind, 16, with_positions=True)
    pos = taken.take_positions()
    assert taken.n_buckets == 8 and not torch.equal(pos.cpu(), torch.arange(g.n_edges, dtype=torch.int32))
    assert call(taken) == 0
    assert torch.equal(out, plain[pos.long()])


def test_own_order_view_of_a_graph(monkeypatch):
    """_lib.own_order_view: the index array in the entry order of the CSR-side work list and the CSC-to-CSR map between the
    two entry orders.  Per-edge tensors kept in that order give the same multi-head SpMM (through the map) and SDDMM as the
    caller's order gives, bit for bit; rows keep their entries; the view is cached; plain lists give the arrays back."""
    from ae_mlsys_gnn_amd import _lib
    from ae_mlsys_gnn_amd.operators.mhspmm import mhsddmm, mhspmm
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "1")
    monkeypatch.setenv("FGNN_BUCKET_MIN_DEG", "16")
    _lib.clear_schedule_cache()
    g = graphs.add_csc_torch(graphs.rmat_graph(1500, 90000, seed=5)).to(DEV)
    idx_own, perm_own = _lib.own_order_view(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute)
    pos_r = _lib.edge_positions(g.row_ptr, g.col_ind)
    assert pos_r is not None and torch.equal(idx_own, g.col_ind[pos_r.long()])
    rows = torch.repeat_interleave(torch.arange(g.n, device=DEV), (g.row_ptr[1:] - g.row_ptr[:-1]).long())
    assert torch.equal(rows[pos_r.long()], rows)                       # a row's entries stay in the row
    assert torch.equal(torch.sort(perm_own).values, torch.arange(g.n_edges, dtype=torch.int32, device=DEV))
    again = _lib.own_order_view(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute)
    assert again[0].data_ptr() == idx_own.data_ptr() and again[1].data_ptr() == perm_own.data_ptr()
    h, f = 4, 16
    torch.manual_seed(0)
    w = torch.randn(g.n_edges, h, device=DEV)
    a, b = torch.randn(g.n, h, f, device=DEV), torch.randn(g.n, h, f, device=DEV)
    w_own = w[pos_r.long()].contiguous()
    assert torch.equal(mhspmm(g.row_ptr, g.col_ind, w_own, a, own_order=True), mhspmm(g.row_ptr, g.col_ind, w, a))
    assert torch.equal(mhspmm(g.col_ptr, g.row_ind, w_own, a, pos_map=perm_own, own_order=True),
                       mhspmm(g.col_ptr, g.row_ind, w, a, pos_map=g.permute))
    assert torch.equal(mhsddmm(g.row_ptr, g.col_ind, a, b, own_order=True), mhsddmm(g.row_ptr, g.col_ind, a, b)[pos_r.long()])
    monkeypatch.setenv("FGNN_XCD_BUCKETS", "0")
    _lib.clear_schedule_cache()
    idx_p, perm_p = _lib.own_order_view(g.row_ptr, g.col_ind, g.col_ptr, g.row_ind, g.permute)
    assert idx_p.data_ptr() == g.col_ind.data_ptr() and perm_p.data_ptr() == g.permute.data_ptr()
    _lib.clear_schedule_cache()

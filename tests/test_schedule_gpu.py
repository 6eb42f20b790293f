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
        out.append((s.n_items, s.n_partials, s.n_edges, items.cpu(), splits.cpu(), None if pos is None else pos.cpu(), s.device_bytes()))
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

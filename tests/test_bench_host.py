"""CPU-side checks of bench.py's host logic: the one-GPU contract, the roofline record, the byte-count file and the
row sampler of the CPU baselines.  Nothing here touches a GPU."""
import json
import os
import subprocess
import sys
import warnings

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402
from ae_mlsys_gnn_amd import graphs  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode == 2
    assert "ONE GPU" in res.stderr and res.stdout.strip() == ""
    env = dict(os.environ, WORLD_SIZE="4")
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True, env=env)
    assert res.returncode == 2 and "ONE GPU" in res.stderr


def test_roofline_record_is_measured_bytes_when_there_are_some():
    rec = bench.roofline_record("k", alg_bytes=100e9, ms=10.0, traffic=40e9)
    assert rec["achieved"] == 4000.0 and rec["frac"] == 0.5 and rec["peak"] == 8000.0 and rec["unit"] == "GB/s" and rec["bound"] == "hbm"
    assert rec["effective_gather_GBps"] == 10000.0 and "measured" in rec["achieved_basis"]
    assert "traffic_stale" not in rec
    assert bench.roofline_record("k", 100e9, 10.0, 40e9, stale=True)["traffic_stale"] is True
    rec = bench.roofline_record("k", alg_bytes=16e9, ms=4.0, traffic=None)
    assert rec["traffic"] is None and rec["achieved"] == 4000.0 and "algorithmic" in rec["achieved_basis"]


def test_byte_count_file_names_every_entry_point_bench_reads():
    with open(bench.TRAFFIC_FILE) as fh:
        t = json.load(fh)
    w = t["workloads"]
    for wl in ("gat_c2", "gat_c5_layer1", "gat_c5_layer2"):
        assert {"fwd", "bwd", "stash_bwd", "stash_writer"} <= set(w[wl]), wl
    assert {"fwd", "bwd", "bwd_summed"} <= set(w["gmm_c4"]) and {"fwd", "bwd", "bwd_blocked"} <= set(w["edgeconv_c3"])
    assert {"u_add_v", "u_add_v_backward", "edge_softmax", "edge_softmax_backward", "mhsddmm", "mhtranspose", "gat_scatter",
            "gat_gather_row"} <= set(w["small_ops_c2"])
    assert all(isinstance(v, int) and v > 0 for d in w.values() for v in d.values())
    assert len(t["csrc_sha256"]) == 64 and "FETCH_SIZE" in t["how"]
    traffic, stale = bench.measured_traffic("gat_c2")
    assert traffic == w["gat_c2"]
    if stale:          # bench.py prints the same warning and marks its records `traffic_stale`
        warnings.warn("profiles/traffic.json was measured at other kernel sources than the present ones")


def test_stale_byte_counts_are_flagged(tmp_path, monkeypatch):
    f = tmp_path / "traffic.json"
    f.write_text(json.dumps({"csrc_sha256": "0" * 64, "measured_at_commit": "abc", "workloads": {"gat_c2": {"fwd": 1}}}))
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(f))
    traffic, stale = bench.measured_traffic("gat_c2")
    assert traffic == {"fwd": 1} and stale is True
    f.write_text(json.dumps({"csrc_sha256": bench.csrc_digest(), "workloads": {}}))
    assert bench.measured_traffic("gat_c2") == (None, False)
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(tmp_path / "missing.json"))
    assert bench.measured_traffic("gat_c2") == (None, False)


def test_row_sample_of_the_cpu_baselines_keeps_whole_rows():
    g = graphs.add_csc_torch(graphs.rmat_graph(500, 6000, seed=3))
    rp_s, ci_s, e_s, r = bench.sample_rows_subgraph(g, 1500)
    rp, ci = g.row_ptr.long(), g.col_ind
    deg, deg_s = rp[1:] - rp[:-1], rp_s.long()[1:] - rp_s.long()[:-1]
    assert rp_s.numel() == g.n + 1 and int(rp_s[0]) == 0 and int(rp_s[-1]) == e_s == ci_s.numel()
    kept = deg_s > 0
    assert torch.equal(deg_s[kept], deg[kept]) and int(kept.sum()) <= r <= g.n and e_s >= 1500
    for row in torch.nonzero(kept).flatten()[:50].tolist():          # a sampled row keeps its sources in their order
        assert torch.equal(ci_s[int(rp_s[row]):int(rp_s[row + 1])], ci[int(rp[row]):int(rp[row + 1])])

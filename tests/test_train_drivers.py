"""Training drivers (ae_mlsys_gnn_amd.train): host-side data handling on the CPU, short end-to-end
runs of the three drivers on the GPU."""
import os

import numpy as np
import pytest
import torch

from ae_mlsys_gnn_amd import graphs

DEV = "cuda:0"


# ------------------------------------------------------------------ host side (no GPU)
def test_node_dataset_files_are_found_and_parsed(tmp_path):
    import scipy.sparse as sp
    from ae_mlsys_gnn_amd.train import datasets
    rng = np.random.default_rng(0)
    n, e = 30, 100
    src, dst = rng.integers(0, n, e), rng.integers(0, n, e)
    feat, label = rng.standard_normal((n, 5)).astype(np.float32), rng.integers(0, 4, n)
    tr = np.arange(n) < 20
    np.savez(tmp_path / "cora.npz", src=src, dst=dst, feat=feat, label=label, train_mask=tr, val_mask=~tr, test_mask=~tr)
    got = datasets._read_node_files("cora", str(tmp_path))
    assert got is not None and torch.equal(got[0], torch.from_numpy(src)) and got[2].dtype == torch.float32 and got[4].sum() == 20
    assert datasets._read_node_files("pubmed", str(tmp_path)) is None and datasets._read_node_files("cora", None) is None
    # the layout of DGL's Reddit download
    os.makedirs(tmp_path / "reddit")
    sp.save_npz(tmp_path / "reddit" / "reddit_graph.npz", sp.coo_matrix((np.ones(e), (src, dst)), shape=(n, n)))
    types = rng.integers(1, 4, n)
    np.savez(tmp_path / "reddit" / "reddit_data.npz", feature=feat, label=label, node_types=types)
    r = datasets._read_node_files("reddit", str(tmp_path))
    assert sorted(zip(r[0].tolist(), r[1].tolist())) == sorted(zip(src.tolist(), dst.tolist()))
    assert torch.equal(r[4], torch.from_numpy(types == 1)) and torch.equal(r[6], torch.from_numpy(types == 3))
    with pytest.raises(ValueError, match="Unknown dataset"):
        datasets.load_node_dataset("nope", "cpu")


def test_graph_cache_round_trip_and_point_cloud_files(tmp_path):
    from ae_mlsys_gnn_amd.train import datasets
    g = graphs.add_csc_torch(graphs.uniform_graph(50, 300, seed=1))
    datasets.save_graph(str(tmp_path / "g.npz"), g)
    h = datasets.load_graph(str(tmp_path / "g.npz"), "cpu")
    assert h.n == g.n and all(torch.equal(getattr(g, k), getattr(h, k)) for k in ("row_ptr", "col_ind", "col_ptr", "row_ind", "permute"))
    np.savez(tmp_path / "bad.npz", n=np.int64(50), row_ptr=g.row_ptr.numpy()[:-1], col_ind=g.col_ind.numpy(), col_ptr=g.col_ptr.numpy(),
             row_ind=g.row_ind.numpy(), permute=g.permute.numpy())
    with pytest.raises(ValueError, match="entries, expected"):
        datasets.load_graph(str(tmp_path / "bad.npz"), "cpu")
    data = np.random.default_rng(0).standard_normal((6, 40, 3)).astype(np.float32)
    np.savez(tmp_path / "clouds.npz", data=data, label=np.array([[0], [3], [1], [2], [3], [0]]))
    c = datasets.load_point_clouds("cpu", str(tmp_path / "clouds.npz"), n_points=32)
    assert c.data.shape == (6, 32, 3) and c.label.tolist() == [0, 3, 1, 2, 3, 0] and c.n_classes == 4
    s = datasets.load_point_clouds("cpu", None, n_clouds=5, n_points=16)
    assert s.source == "synthetic" and s.data.shape == (5, 16, 3) and float(s.data.abs().max()) <= 1
    with pytest.raises(RuntimeError, match="h5py"):
        datasets.load_point_clouds("cpu", str(tmp_path / "clouds.h5"))


def test_malformed_graphs_are_rejected_on_the_host_before_any_kernel(tmp_path):
    """Node ids outside [0, n), int64 ids that an int32 cast would wrap into range, broken pointer arrays and
    permutations: the loaders raise ValueError from host-side reductions; nothing is handed to the device (the
    target device here is the CPU, which the operators refuse, so reaching them would raise FgnnError instead)."""
    from ae_mlsys_gnn_amd.train import datasets
    n = 20
    src = torch.arange(n, dtype=torch.int64)
    dst = torch.flip(src, [0])
    for bad_src, bad_dst, msg in ((src.clone().index_fill_(0, torch.tensor([3]), n), dst, r"src ids must lie in \[0, 20\)"),
                                  (src, dst.clone().index_fill_(0, torch.tensor([0]), -1), r"dst ids must lie"),
                                  (src.clone().index_fill_(0, torch.tensor([5]), (1 << 32) + 4), dst, r"src ids must lie"),   # wraps to 4 as int32
                                  (src.double(), dst, "integer array"), (src[:-1], dst, "sources for")):
        with pytest.raises(ValueError, match=msg):
            datasets.graph_from_edges(bad_src, bad_dst, n, "cpu")
    g = graphs.add_csc_torch(graphs.uniform_graph(n, 90, seed=2))
    good = {k: getattr(g, k).numpy().copy() for k in ("row_ptr", "col_ind", "col_ptr", "row_ind", "permute")}
    graphs.validate_graph(g)

    def broken(key, fn, match):
        arr = {k: v.copy() for k, v in good.items()}
        fn(arr[key])
        np.savez(tmp_path / "b.npz", n=np.int64(n), **arr)
        with pytest.raises(ValueError, match=match):
            datasets.load_graph(str(tmp_path / "b.npz"), "cpu")

    def set_(i, v):
        def f(a):
            a[i] = v
        return f
    broken("col_ind", set_(7, n), "node ids must lie")
    broken("row_ind", set_(0, -2), "node ids must lie")
    broken("row_ptr", set_(3, good["row_ptr"][4] + 1), "never decrease")
    broken("row_ptr", set_(0, 1), "start at 0")
    broken("col_ptr", set_(n, good["col_ptr"][n] + 5), "end at E")
    broken("permute", set_(2, g.n_edges), "permute entries")
    arr = dict(good, col_ind=good["col_ind"].astype(np.float32))
    np.savez(tmp_path / "b.npz", n=np.int64(n), **arr)
    with pytest.raises(ValueError, match="integer arrays"):
        datasets.load_graph(str(tmp_path / "b.npz"), "cpu")
    # the C-ABI check refuses bad sizes without a GPU (its kernel path is covered by the GPU tests)
    from ae_mlsys_gnn_amd import _lib
    assert _lib.lib().fgnn_validate_graph(None, None, 4, 4, 3, None) == -1
    assert _lib.lib().fgnn_schedule_device_bytes(None) == 0


def test_driver_command_lines_and_loss():
    """The flags of the reference's scripts parse (script/train/train_gatconv_our.py:212-243,
    train_gmmconv_our.py:199-221, train_edgeconv_our.py:153-162); the smoothed loss equals its
    one-hot definition (train_edgeconv_our.py:76-82)."""
    from ae_mlsys_gnn_amd.train import train_edgeconv, train_gatconv, train_gmmconv
    a = train_gatconv.build_parser().parse_args("--dataset=reddit --num-heads=4 --num-hidden=64 --epochs=100 --num-layers 1 --num-out-heads 1 "
                                                "--lr 0.005 --weight-decay 5e-4 --negative-slope 0.2 --gpu 0 --output figure10.csv".split())
    assert (a.dataset, a.num_heads, a.num_hidden, a.epochs, a.variant) == ("reddit", 4, 64, 100, "our")
    m = train_gmmconv.build_parser().parse_args("--dataset=pubmed --n-epochs=100 --n-hidden=16 --n-kernels=3 --pseudo-dim=3 --dropout 0.5".split())
    assert (m.n_kernels, m.pseudo_dim, m.n_layers) == (3, 3, 0)
    e = train_edgeconv.build_parser().parse_args("--k=20 --batch-size=32 --num-epochs 10 --dataset-path x.h5".split())
    assert (e.k, e.batch_size) == (20, 32)
    torch.manual_seed(0)
    logits, y = torch.randn(7, 5, dtype=torch.float64), torch.randint(0, 5, (7,))
    one_hot = torch.zeros(7, 5, dtype=torch.float64).scatter_(1, y.view(-1, 1), 1.0)
    target = one_hot * 0.8 + (1 - one_hot) * 0.2 / 4
    want = -(target * torch.log_softmax(logits, 1)).sum(1).mean()
    assert abs(float(train_edgeconv.compute_loss(logits, y)) - float(want)) < 1e-12


# ------------------------------------------------------------------ on the GPU
@pytest.mark.gpu
def test_graph_from_edges_matches_scipy():
    import scipy.sparse as sp
    from ae_mlsys_gnn_amd.train import datasets
    rng = np.random.default_rng(3)
    n, e = 500, 6000
    src, dst = rng.integers(0, n, e), rng.integers(0, n, e)
    g = datasets.graph_from_edges(torch.from_numpy(src), torch.from_numpy(dst), n, DEV, dedupe=True)
    keep = src != dst
    a = sp.coo_matrix((np.ones(keep.sum() + n), (np.r_[dst[keep], np.arange(n)], np.r_[src[keep], np.arange(n)])), shape=(n, n)).tocsr()
    a.sum_duplicates(); a.sort_indices()
    assert np.array_equal(g.row_ptr.cpu().numpy(), a.indptr) and np.array_equal(g.col_ind.cpu().numpy(), a.indices)
    csc = sp.csr_matrix((np.arange(a.nnz), a.indices, a.indptr), shape=(n, n)).tocsc()
    assert np.array_equal(g.col_ptr.cpu().numpy(), csc.indptr) and np.array_equal(g.row_ind.cpu().numpy(), csc.indices)
    assert np.array_equal(g.permute.cpu().numpy(), csc.data)
    # duplicates kept as independent edges without dedupe
    g2 = datasets.graph_from_edges(torch.tensor([1, 1, 2]), torch.tensor([0, 0, 0]), 3, DEV)
    assert g2.n_edges == 6 and g2.col_ind.tolist()[:3] == [0, 1, 1]
    p = datasets.degree_pseudo(g2)                      # rows: node 0 has in-degree 4, nodes 1, 2 have 1
    assert torch.allclose(p[:4].cpu(), torch.tensor([[0.5, 0.5], [1, 0.5], [1, 0.5], [1, 0.5]]))


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["our", "stash", "fusescatter"])
def test_gat_driver_trains(tmp_path, variant):
    from ae_mlsys_gnn_amd.train import train_gatconv
    out = tmp_path / "rows.csv"
    r = train_gatconv.main(["--dataset", "cora", "--num-heads", "2", "--num-hidden", "16", "--epochs", "15", "--warmup", "2",
                            "--variant", variant, "--output", str(out), "--lr", "0.01"])
    assert r["source"] == "synthetic" and r["nodes"] == 2708 and r["last_loss"] < r["first_loss"]
    assert out.read_text().startswith("train_GAT_%s,dataset=cora,head=2,f=16,latency=" % variant)


@pytest.mark.gpu
def test_gat_driver_reads_files_and_caches_graph(tmp_path):
    from ae_mlsys_gnn_amd.train import train_gatconv
    rng = np.random.default_rng(0)
    n, e = 400, 3000
    label = rng.integers(0, 3, n)
    feat = (np.eye(3)[label] + 0.1 * rng.standard_normal((n, 3))).astype(np.float32)       # learnable from the features
    tr = rng.random(n) < 0.5
    src = rng.integers(0, n, e)
    same = [np.flatnonzero(label == c) for c in range(3)]
    dst = np.array([rng.choice(same[label[s]]) for s in src])                               # edges stay inside a class
    np.savez(tmp_path / "citeseer.npz", src=src, dst=dst, feat=feat, label=label, train_mask=tr, val_mask=~tr, test_mask=~tr)
    argv = ["--dataset", "citeseer", "--data-root", str(tmp_path), "--cache-dir", str(tmp_path / "cache"), "--num-hidden", "8",
            "--epochs", "60", "--warmup", "0", "--output", "", "--lr", "0.02"]
    r = train_gatconv.main(argv)
    assert r["source"].startswith("file:") and r["nodes"] == n and r["test_acc"] > 0.8
    assert len(os.listdir(tmp_path / "cache")) == 1
    r2 = train_gatconv.main(argv)                       # second run takes the cached arrays
    assert r2["edges"] == r["edges"] and abs(r2["last_loss"] - r["last_loss"]) < 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["our", "stash"])
def test_monet_driver_trains(tmp_path, variant):
    from ae_mlsys_gnn_amd.train import train_gmmconv
    out = tmp_path / "rows.csv"
    r = train_gmmconv.main(["--dataset", "pubmed", "--scale", "0.2", "--n-epochs", "15", "--n-kernels", "3", "--pseudo-dim", "3",
                            "--dropout", "0", "--variant", variant, "--output", str(out)])
    assert r["last_loss"] < r["first_loss"]
    assert out.read_text().startswith("train_monet_%s,dataset=pubmed,k=3,d=3,latency=" % variant)


@pytest.mark.gpu
@pytest.mark.parametrize("knn", ["fgnn", "torch"])
def test_dgcnn_driver_trains(tmp_path, knn):
    """Four shape classes (cube, sphere shell, segment, two blobs) that survive the scale/shift
    augmentation: the DGCNN has to separate them within a few epochs."""
    from ae_mlsys_gnn_amd.train import train_edgeconv
    rng = np.random.default_rng(1)
    m, p = 80, 128
    label = np.arange(m) % 4
    data = np.empty((m, p, 3), np.float32)
    for i, c in enumerate(label):
        u = rng.uniform(-1, 1, (p, 3))
        if c == 1:
            u = rng.standard_normal((p, 3)); u /= np.linalg.norm(u, axis=1, keepdims=True)
        elif c == 2:
            u = np.outer(rng.uniform(-1, 1, p), rng.standard_normal(3)) + 0.01 * rng.standard_normal((p, 3))
        elif c == 3:
            u = 0.1 * rng.standard_normal((p, 3)) + np.where(rng.random((p, 1)) < 0.5, 0.7, -0.7)
        data[i] = u
    np.savez(tmp_path / "clouds.npz", data=data, label=label)
    out = tmp_path / "rows.csv"
    r = train_edgeconv.main(["--dataset-path", str(tmp_path / "clouds.npz"), "--k", "8", "--batch-size", "16", "--num-points", "128",
                             "--num-epochs", "12", "--warmup-epochs", "0", "--knn", knn, "--output", str(out)])
    assert r["source"].startswith("file:") and r["iters_per_epoch"] == 4 and all(np.isfinite(r["losses"]))
    # SGD at lr 0.1 with dropout: the loss is noisy, the accuracy (chance = 0.25) is the stable signal
    assert np.mean(r["train_acc"][-3:]) > 0.7 and np.mean(r["train_acc"][-3:]) > r["train_acc"][0], (r["losses"], r["train_acc"])
    assert out.read_text().startswith("train_edgeconv_our,dataset=modelnet40,k=8,batch=16,latency=")


def test_pseudo_projection_equals_linear_tanh():
    from ae_mlsys_gnn_amd.train.train_gmmconv import PseudoProj
    torch.manual_seed(0)
    proj = PseudoProj(2, 3).double()
    x = torch.rand(50, 2, dtype=torch.float64, requires_grad=True)
    want = torch.tanh(torch.nn.functional.linear(x, proj.weight, proj.bias))
    got = proj(x)
    assert torch.allclose(got, want, atol=1e-14)
    gw = torch.autograd.grad(got.sum(), [proj.weight, proj.bias, x])
    ww = torch.autograd.grad(want.sum(), [proj.weight, proj.bias, x])
    assert all(torch.allclose(a, b, atol=1e-12) for a, b in zip(gw, ww))


def test_cross_entropy_helper_equals_torch():
    from ae_mlsys_gnn_amd.train.common import cross_entropy
    torch.manual_seed(0)
    logits = (5 * torch.randn(200, 47, dtype=torch.float64)).requires_grad_(True)
    y = torch.randint(0, 47, (200,))
    want = torch.nn.CrossEntropyLoss()(logits, y)
    got = cross_entropy(logits, y)
    assert abs(float(got.detach()) - float(want.detach())) < 1e-12
    gw, = torch.autograd.grad(want, logits)
    gg, = torch.autograd.grad(got, logits)
    assert torch.allclose(gw, gg, atol=1e-14)


def test_masked_cross_entropy_equals_the_loss_over_the_selected_rows():
    """masked_cross_entropy(logits, MaskedRows(mask, labels)) = CrossEntropyLoss()(logits[mask], labels[mask]) in value
    and gradient (zero on the unselected rows), also when an unselected row carries a placeholder label."""
    from ae_mlsys_gnn_amd.train.common import MaskedRows, masked_cross_entropy
    torch.manual_seed(1)
    logits = (5 * torch.randn(300, 47, dtype=torch.float64)).requires_grad_(True)
    y = torch.randint(0, 47, (300,))
    mask = torch.rand(300) < 0.4
    y_marked = torch.where(mask, y, torch.full_like(y, -1))
    want = torch.nn.CrossEntropyLoss()(logits[mask], y[mask])
    gw, = torch.autograd.grad(want, logits)
    for labels in (y, y_marked):
        got = masked_cross_entropy(logits, MaskedRows(mask, labels))
        assert abs(float(got.detach()) - float(want.detach())) < 1e-12
        gg, = torch.autograd.grad(got, logits)
        assert torch.allclose(gw, gg, atol=1e-14) and float(gg[~mask].abs().max()) == 0.0
    padded = torch.cat([logits.detach(), torch.zeros(300, 1, dtype=torch.float64)], 1)
    assert abs(float(masked_cross_entropy(padded, MaskedRows(mask, y), 47)) - float(want.detach())) < 1e-12


@pytest.mark.gpu
def test_masked_cross_entropy_on_the_device():
    """The same through the fused row pass: padded [N, 48] logits with 47 classes and a cropped view."""
    from ae_mlsys_gnn_amd.train.common import MaskedRows, masked_cross_entropy
    torch.manual_seed(2)
    dev = "cuda:0"
    n, c, width = 5000, 47, 48
    padded = torch.zeros(n, width)
    padded[:, :c] = 4 * torch.randn(n, c)
    y = torch.randint(0, c, (n,))
    mask = torch.rand(n) < 0.3
    ref_in = padded[:, :c].double().requires_grad_(True)
    want = torch.nn.CrossEntropyLoss()(ref_in[mask], y[mask])
    gw, = torch.autograd.grad(want, ref_in)
    rows = MaskedRows(mask.to(dev), torch.where(mask, y, torch.full_like(y, -1)).to(dev))
    for crop in (False, True):
        pd = padded.to(dev).requires_grad_(True)
        got = masked_cross_entropy(pd[:, :c], rows) if crop else masked_cross_entropy(pd, rows, c)
        gg, = torch.autograd.grad(got, pd)
        assert abs(float(got) - float(want)) <= 1e-5 * max(1.0, abs(float(want)))
        assert torch.allclose(gg[:, :c].cpu().double(), gw, rtol=1e-4, atol=1e-9)
        assert float(gg[:, c:].abs().max()) == 0.0 and float(gg[~mask.to(dev)].abs().max()) == 0.0


@pytest.mark.gpu
def test_forward_latency_driver(tmp_path):
    from ae_mlsys_gnn_amd.train import forward_latency
    out = tmp_path / "figure9.csv"
    forward_latency.main(["gat", "--dataset", "cora", "--in_feats", "16", "--out_feats", "6", "--num-heads", "2", "--epochs", "5", "--output", str(out)])
    forward_latency.main(["edgeconv", "--batch-size", "2", "--k", "10", "--epochs", "5", "--output", str(out)])
    forward_latency.main(["monet", "--dataset", "cora", "--n-epochs", "5", "--output", str(out)])
    rows = out.read_text().splitlines()
    assert [r.split(",")[0] for r in rows] == ["gat_with_fusion", "edgeconv_with_fusion", "monet_with_fusion"]
    assert all("latency=" in r and r.endswith("MB") for r in rows)


@pytest.mark.gpu
@pytest.mark.parametrize("model", ["gat", "monet"])
def test_training_step_replays_from_a_hip_graph(model):
    """--hip-graph: the captured step, replayed 12 times with eager work (validation passes, the
    driver's own synchronisations) in between, follows the eager loss trajectory.  The capture is
    preceded by 3 eager steps on a side stream, so 12 replays end where 15 eager steps end."""
    from ae_mlsys_gnn_amd.train import train_gatconv, train_gmmconv
    if model == "gat":
        argv = ["--dataset", "cora", "--num-heads", "2", "--num-hidden", "16", "--warmup", "0", "--output", ""]
        eager, graphed = train_gatconv.main(argv + ["--epochs", "15"]), train_gatconv.main(argv + ["--epochs", "12", "--hip-graph"])
    else:
        argv = ["--dataset", "cora", "--warmup", "0", "--dropout", "0", "--output", ""]
        eager, graphed = train_gmmconv.main(argv + ["--n-epochs", "15"]), train_gmmconv.main(argv + ["--n-epochs", "12", "--hip-graph"])
    assert eager["first_loss"] == graphed["first_loss"]
    # torch's backward of logits[train_idx] adds with atomics, so two eager runs already differ in the
    # last bits and 16 optimizer steps amplify that; a wrong replay would be off by far more
    assert abs(eager["last_loss"] - graphed["last_loss"]) <= 5e-4 * abs(eager["last_loss"]), (eager, graphed)
    assert abs(eager["test_acc"] - graphed["test_acc"]) < 0.02


def test_tall_linear_equals_linear():
    """layers.dense: the chunked reduction over the rows gives the weight gradient of an ordinary Linear
    (row counts that do and do not divide into the chunks, with and without bias / input gradient)."""
    from ae_mlsys_gnn_amd.layers.dense import reduce_over_rows, tall_linear
    torch.manual_seed(0)
    for n, need_gx in ((100, True), (4096 + 17, True), (3 * 2048, False), (70001, True)):
        x = torch.randn(n, 5, dtype=torch.float64, requires_grad=need_gx)
        w = torch.randn(7, 5, dtype=torch.float64, requires_grad=True)
        b = torch.randn(7, dtype=torch.float64, requires_grad=True)
        go = torch.randn(n, 7, dtype=torch.float64)
        for bias in (b, None):
            want = torch.nn.functional.linear(x, w, bias)
            got = tall_linear(x, w, bias)
            assert torch.allclose(got, want, atol=1e-12)
            leaves = [t for t in (x, w, bias) if t is not None and t.requires_grad]
            gw = torch.autograd.grad((want * go).sum(), leaves)
            gg = torch.autograd.grad((got * go).sum(), leaves)
            assert all(torch.allclose(a, c, rtol=1e-10, atol=1e-10) for a, c in zip(gg, gw))
        assert torch.allclose(reduce_over_rows(x.detach(), go), x.detach().t() @ go, rtol=1e-10, atol=1e-10)


def test_column_sum_and_add_bias_equal_the_plain_forms():
    """layers.dense: the chunked column sum (bias gradients of tall matrices) equals g.sum(0) for widths
    that are and are not multiples of 4 and row counts on both sides of the chunking threshold."""
    from ae_mlsys_gnn_amd.layers.dense import add_bias, column_sum
    torch.manual_seed(0)
    for n, c in ((10, 3), (4096, 7), (4096 + 17, 7), (3 * 2048 + 5, 8), (70001, 47), (600000, 64)):
        g = torch.randn(n, c, dtype=torch.float64)
        assert torch.allclose(column_sum(g), g.sum(0), rtol=1e-10, atol=1e-9)
    x = torch.randn(5000, 6, dtype=torch.float64, requires_grad=True)
    b = torch.randn(6, dtype=torch.float64, requires_grad=True)
    go = torch.randn(5000, 6, dtype=torch.float64)
    want = torch.autograd.grad(((x + b) * go).sum(), (x, b))
    got = torch.autograd.grad((add_bias(x, b) * go).sum(), (x, b))
    assert torch.equal(add_bias(x, b), x + b)
    assert all(torch.allclose(a, w, rtol=1e-10, atol=1e-10) for a, w in zip(got, want))


@pytest.mark.gpu
@pytest.mark.parametrize("n,c,width", [(1000, 47, 48), (1000, 47, 47), (513, 7, 7), (300, 10, 12), (77, 200, 200), (64, 1000, 1000), (5, 1, 4),
                                       (2000, 41, 44)])
def test_fused_cross_entropy_rows(n, c, width):
    """The drivers' loss on the GPU (fgnn_cross_entropy_forward / _backward): value and gradient of
    torch.nn.CrossEntropyLoss in float64, for logits that are a [n, c] view of a zero-padded [n, width] array and for
    the padded array itself with the class count handed over; the gradient of the padding columns is zero."""
    from ae_mlsys_gnn_amd.train.common import cross_entropy
    torch.manual_seed(n + c)
    dev = "cuda:0"
    padded = torch.zeros(n, width)
    padded[:, :c] = 4 * torch.randn(n, c)
    y = torch.randint(0, c, (n,))
    ref_in = padded[:, :c].double().requires_grad_(True)
    want = torch.nn.CrossEntropyLoss()(ref_in, y)
    gw, = torch.autograd.grad(want, ref_in)
    pd = padded.to(dev).requires_grad_(True)
    got = cross_entropy(pd, y.to(dev), c)                     # padded array + class count
    gg, = torch.autograd.grad(got, pd)
    assert abs(float(got) - float(want)) <= 1e-5 * max(1.0, abs(float(want)))
    assert torch.allclose(gg[:, :c].cpu().double(), gw, rtol=1e-4, atol=1e-7)
    assert float(gg[:, c:].abs().max()) == 0.0 if width > c else True
    pv = padded.to(dev).requires_grad_(True)
    got2 = cross_entropy(pv[:, :c], y.to(dev))                # a cropped view, read in place
    gg2, = torch.autograd.grad(got2, pv)
    assert abs(float(got2) - float(want)) <= 1e-5 * max(1.0, abs(float(want)))
    assert torch.allclose(gg2[:, :c].cpu().double(), gw, rtol=1e-4, atol=1e-7)
    # a label outside [0, c) reads nothing and poisons the loss
    bad = y.clone(); bad[0] = c
    assert torch.isnan(cross_entropy(padded.to(dev), bad.to(dev), c))

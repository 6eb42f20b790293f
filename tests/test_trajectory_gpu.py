"""Training-trajectory parity: the models of the reference's training scripts stepped on the HIP path
(fp32, the package's layers and the drivers' model classes) next to float64 CPU models assembled from
the oracle's layer functions, from the same initial weights, on the same seeded data.

  GAT    script/train/train_gatconv_our.py:33-53 (hidden GATConv flattened, output GATConv averaged over
         its heads), CrossEntropyLoss on the training nodes, Adam(lr 5e-3, weight decay 5e-4) (:166-167);
         recompute and stash variants must both follow the float64 trajectory.
  MoNet  script/train/train_gmmconv_our.py:46-75 (GMMConv layers, each with Linear(2, dim) + Tanh on the
         degree pseudo-coordinates), Adam; dropout 0 so that both sides see the same network.
  DGCNN  the EdgeConv stack of script/train/train_edgeconv_our.py:44-60 (kNN graph rebuilt from each
         layer's input, LeakyReLU(0.2)), two layers, max-pooled per cloud into a linear classifier,
         SGD(0.1, momentum 0.9, weight decay 1e-4) (:204).  The float64 side walks the graphs the GPU
         side built (a neighbour list is data: a near-tie in a distance must not fork the two runs).

Checked: the loss of every step within rel 1e-4, and the weights after the last step.  Adam divides the
gradient by its running magnitude, so a weight whose gradient is at rounding level moves by about +-lr
per step whatever the gradient's exact value: for Adam the final weights are compared through the
update they received, ||w_hip - w_ref|| <= 1e-3 ||w_ref - w_init|| per tensor; SGD's update is linear
in the gradient, there every tensor is compared at 1e-4 of its largest entry."""
import copy

import pytest
import torch
from torch import nn

from oracle import fgnn_oracle as orc
from ae_mlsys_gnn_amd import graphs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
STEPS = 10


def _check_losses(got, want, what):
    for t, (a, b) in enumerate(zip(got, want)):
        assert abs(a - b) <= 1e-4 * abs(b), "%s: loss of step %d is %.8f, float64 model has %.8f" % (what, t, a, b)


def _check_adam_weights(model, ref_params, init_params, what):
    for (name, p), r, w0 in zip(model.named_parameters(), ref_params, init_params):
        moved = float((r.detach() - w0).norm())
        diff = float((p.detach().cpu().double() - r.detach()).norm())
        assert diff <= 1e-3 * moved + 1e-7, "%s: %s ended %.3e away from the float64 weights after an update of norm %.3e" % (what, name, diff, moved)


# ------------------------------------------------------------------------------------------------ GAT
class _GatRef:
    """Float64 twin of train_gatconv.GAT: same parameter order (per layer W, attn_l, attn_r)."""

    def __init__(self, model):
        self.params = [p.detach().cpu().double().clone().requires_grad_(True) for p in model.parameters()]
        self.slopes = [l.negative_slope for l in list(model.hidden) + [model.out]]

    def forward(self, g, x):
        h = x
        n_layers = len(self.params) // 3
        for l in range(n_layers):
            w, al, ar = self.params[3 * l: 3 * l + 3]
            h = orc.gat_layer_ours(w, al, ar, g.row_ptr, g.col_ind, self.slopes[l], h)
            h = h.flatten(1) if l < n_layers - 1 else h.mean(1)
        return h


@pytest.mark.parametrize("variant", ["our", "stash"])
def test_gat_training_trajectory_matches_float64_model(variant):
    from ae_mlsys_gnn_amd.train import common
    from ae_mlsys_gnn_amd.train.train_gatconv import GAT, VARIANTS
    torch.manual_seed(0)
    g = graphs.add_csc_torch(graphs.rmat_graph(5000, 60000, seed=3))
    n, fin, hidden, heads, classes = g.n, 48, 16, 4, 7
    gen = torch.Generator().manual_seed(1)
    feat = torch.randn(n, fin, generator=gen)
    label = torch.randint(0, classes, (n,), generator=gen)
    train_idx = (torch.rand(n, generator=gen) < 0.6).nonzero().squeeze(1)
    model = GAT(VARIANTS[variant], 1, fin, hidden, classes, [heads, 1], 0.2)
    ref = _GatRef(model)
    init = [p.detach().clone() for p in ref.params]
    ref_opt = torch.optim.Adam(ref.params, lr=5e-3, weight_decay=5e-4)
    ref_losses = []
    for _ in range(STEPS):
        loss = nn.functional.cross_entropy(ref.forward(g, feat.double())[train_idx], label[train_idx])
        ref_opt.zero_grad()
        loss.backward()
        ref_opt.step()
        ref_losses.append(float(loss.detach()))
    model = model.to(DEV)
    gd = g.to(DEV)
    opt = torch.optim.Adam(model.parameters(), lr=5e-3, weight_decay=5e-4)
    fd, ld, td = feat.to(DEV), label.to(DEV), train_idx.to(DEV)
    extra = True if variant == "our" else gd.permute
    losses = []
    for _ in range(STEPS):
        loss = common.cross_entropy(model(gd, fd, extra)[td], ld[td])
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert ref_losses[-1] < ref_losses[0]
    _check_losses(losses, ref_losses, "GAT (%s)" % variant)
    _check_adam_weights(model, ref.params, init, "GAT (%s)" % variant)


# ------------------------------------------------------------------------------------------------ MoNet
class _MonetRef:
    """Float64 twin of train_gmmconv.MoNet without residuals: per layer (mu, inv_sigma, fc.weight, bias),
    then per layer the pseudo projection (weight, bias), in the order of model.parameters()."""

    def __init__(self, model):
        self.names = [n for n, _ in model.named_parameters()]
        self.params = [p.detach().cpu().double().clone().requires_grad_(True) for p in model.parameters()]
        self.n_layers = len(model.layers)

    def _p(self, name):
        return self.params[self.names.index(name)]

    def forward(self, g, feat, pseudo):
        h = feat
        for i in range(self.n_layers):
            ps = torch.tanh(nn.functional.linear(pseudo, self._p("pseudo_proj.%d.weight" % i), self._p("pseudo_proj.%d.bias" % i)))
            h = orc.gmm_layer_dgl(self._p("layers.%d.fc.weight" % i), self._p("layers.%d.mu" % i), self._p("layers.%d.inv_sigma" % i),
                                  self._p("layers.%d.bias" % i), g.row_ptr, g.col_ind, h, ps)
        return h


@pytest.mark.parametrize("variant,csc_pseudo", [("our", 2), ("our", 0), ("stash", 2)])
def test_monet_training_trajectory_matches_float64_model(variant, csc_pseudo):
    """K = 2, dim = 1 (the reddit rows of the reference's figure 7), two layers: the first transforms before
    aggregating, the second aggregates first (16 -> 2 x 7); with the per-edge data in the schedules' own orders
    (the drivers' default) and as one CSR-ordered copy (the reference's data flow)."""
    from ae_mlsys_gnn_amd.train import common, datasets
    from ae_mlsys_gnn_amd.train.train_gmmconv import MoNet, VARIANTS, schedule_order_copies
    torch.manual_seed(0)
    g = graphs.add_csc_torch(graphs.rmat_graph(4000, 50000, seed=5))
    n, fin, hidden, classes = g.n, 40, 16, 7
    gen = torch.Generator().manual_seed(2)
    feat = torch.randn(n, fin, generator=gen) * 0.05        # the sum aggregator adds up to ~2000 neighbours on the hubs
    label = torch.randint(0, classes, (n,), generator=gen)
    train_idx = (torch.rand(n, generator=gen) < 0.6).nonzero().squeeze(1)
    pseudo = datasets.degree_pseudo(g)
    model = MoNet(VARIANTS[variant], fin, hidden, classes, 0, 1, 2, 0.0)
    ref = _MonetRef(model)
    init = [p.detach().clone() for p in ref.params]
    ref_opt = torch.optim.Adam(ref.params, lr=1e-2, weight_decay=5e-4)
    ref_losses = []
    for _ in range(STEPS):
        loss = nn.functional.cross_entropy(ref.forward(g, feat.double(), pseudo.double())[train_idx], label[train_idx])
        ref_opt.zero_grad()
        loss.backward()
        ref_opt.step()
        ref_losses.append(float(loss.detach()))
    model = model.to(DEV)
    gd = g.to(DEV)
    pd = pseudo.to(DEV)
    own_order = csc_pseudo == 2
    pcsc = None
    if own_order:
        pd, pcsc = schedule_order_copies(gd, pd)
    opt = torch.optim.Adam(model.parameters(), lr=1e-2, weight_decay=5e-4)
    fd, ld, td = feat.to(DEV), label.to(DEV), train_idx.to(DEV)
    losses = []
    for _ in range(STEPS):
        loss = common.cross_entropy(model(gd, fd, pd, pcsc, own_order=own_order)[td], ld[td])
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert ref_losses[-1] < ref_losses[0]
    _check_losses(losses, ref_losses, "MoNet (%s, csc_pseudo=%d)" % (variant, csc_pseudo))
    _check_adam_weights(model, ref.params, init, "MoNet (%s, csc_pseudo=%d)" % (variant, csc_pseudo))


# ------------------------------------------------------------------------------------------------ EdgeConv stack
class _EdgeStack(nn.Module):
    """Two EdgeConv layers on kNN graphs rebuilt from each layer's input, LeakyReLU(0.2) after each, the two
    outputs concatenated, max-pooled per cloud and classified by one Linear.  `graphs_in`: neighbour lists to
    walk instead of building them (the float64 twin gets the GPU side's); the lists used are kept in .graphs."""

    def __init__(self, k, dims, classes, conv_cls, knn):
        super().__init__()
        self.k, self.knn = k, knn
        self.conv = nn.ModuleList(conv_cls(dims[i], dims[i + 1]) for i in range(len(dims) - 1))
        self.out = nn.Linear(sum(dims[1:]), classes)
        self.graphs = []

    def forward(self, x, graphs_in=None):
        b, p, _ = x.shape
        h, hs = x, []
        self.graphs = []
        for i, conv in enumerate(self.conv):
            src = self.knn(h.detach(), self.k) if graphs_in is None else graphs_in[i]
            self.graphs.append(src)
            h = nn.functional.leaky_relu(conv(self.k, src, h.reshape(b * p, -1), block=p), 0.2).view(b, p, -1)
            hs.append(h)
        return self.out(torch.cat(hs, 2).max(1).values)


class _EdgeConvRef(nn.Module):
    """EdgeConv_reorg (layers/edgeconv_layer.py:102-109) on the oracle's differentiable form."""

    def __init__(self, in_feat, out_feat):
        super().__init__()
        self.theta = nn.Linear(in_feat, out_feat, bias=False)
        self.phi = nn.Linear(in_feat, out_feat, bias=False)

    def forward(self, k, src_ind, feat, block=None):
        h_src = self.theta(feat)
        return orc.edgeconv_forward_autograd(k, src_ind, h_src, self.phi(feat) - h_src)


def test_edgeconv_stack_training_trajectory_matches_float64_model():
    from ae_mlsys_gnn_amd.layers import EdgeConv
    from ae_mlsys_gnn_amd.operators.knn import knn_graph
    torch.manual_seed(0)
    b, p, k, classes = 6, 128, 10, 5
    gen = torch.Generator().manual_seed(4)
    clouds = torch.rand(b, p, 3, generator=gen) * 2 - 1
    label = torch.randint(0, classes, (b,), generator=gen)
    model = _EdgeStack(k, [3, 32, 32], classes, EdgeConv, knn_graph)
    ref = _EdgeStack(k, [3, 32, 32], classes, _EdgeConvRef, None)
    ref.load_state_dict(copy.deepcopy(model.state_dict()))
    ref = ref.double()
    model = model.to(DEV)
    opt = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9, weight_decay=1e-4)
    ref_opt = torch.optim.SGD(ref.parameters(), lr=0.1, momentum=0.9, weight_decay=1e-4)
    xd, yd = clouds.to(DEV), label.to(DEV)
    losses, ref_losses = [], []
    for _ in range(STEPS):
        loss = nn.functional.cross_entropy(model(xd), yd)
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
        rloss = nn.functional.cross_entropy(ref(clouds.double(), [s.cpu() for s in model.graphs]), label)
        ref_opt.zero_grad()
        rloss.backward()
        ref_opt.step()
        ref_losses.append(float(rloss.detach()))
    assert ref_losses[-1] < ref_losses[0]
    _check_losses(losses, ref_losses, "EdgeConv stack")
    for (name, pg), pr in zip(model.named_parameters(), ref.parameters()):
        diff = float((pg.detach().cpu().double() - pr.detach()).abs().max())
        assert diff <= 1e-4 * float(pr.detach().abs().max()), "EdgeConv stack: %s differs from the float64 weights by %.3e" % (name, diff)

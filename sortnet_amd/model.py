"""The distance-layer stack that the benchmark times and tests/test_gpu_bench_stack.py checks against the oracle: the `fc_dist`
part of the reference's SortMLPModel (ell_inf_models.py:17-50) -- `depth - 1` distance layers of
equal width with mean shift, then a distance layer onto the classes with a bias -- and the
reference's hinge loss on the 1-Lipschitz margin (main.py:329-335, ell_inf_models.py:45-50).

Training forward uses the fused masked order-statistic neuron (keep probability q) where the
reference registers a dropout rate, i.e. on every layer but the first (ell_inf_models.py:24-27);
`bounds()` is the certification pass: interval bounds through the l-inf form of every layer
(main.py:205-240 with q = 1), mean shift taken from the running means.
"""
import torch

from . import functional as F
from .ext import MASK_TERM
from .losses import hinge_loss  # noqa: F401  (the benchmark's loss)


class DistanceMLP:
    def __init__(self, in_features, width, depth, num_classes, q=0.3, device="cuda", seed=0, mask_mode=MASK_TERM,
                 momentum=0.1, weight_std=None):
        """weight_std: standard deviation of the initial weights; None = fan_in ** -0.5 (the scale the benchmark
        configurations state for single layers), 1.0 = the reference's own initialisation (core/models/norm_dist.py:30)."""
        g = torch.Generator().manual_seed(seed)
        dims = [in_features] + [width] * (depth - 1) + [num_classes]
        self.weights = []
        for fan_in, fan_out in zip(dims[:-1], dims[1:]):
            w = torch.randn(fan_out, fan_in, generator=g) * (fan_in ** -0.5 if weight_std is None else weight_std)
            self.weights.append(w.to(device).requires_grad_())
        self.bias = torch.zeros(num_classes, device=device, requires_grad=True)
        self.running_mean = [torch.zeros(d, device=device) for d in dims[1:-1]]
        self.q, self.mask_mode, self.momentum = q, mask_mode, momentum
        self.num_layers = len(self.weights)

    def parameters(self):
        return self.weights + [self.bias]

    def terms_per_sample(self):
        return sum(w.numel() for w in self.weights)

    def forward(self, x, step_seed, trace=None, after_layer=None, before_layer=None):
        """Training forward: x (B, in_features) -> distances to the class prototypes (B, classes).
        `trace`, a list, receives per layer (input, raw distances, batch mean or None) for inspection;
        `before_layer(i)` is called before anything that reads layer i's weight (or, on the last layer, the bias) is
        queued, `after_layer(i, weight)` right after layer i's distance op has been queued."""
        h = x.unsqueeze(-1)
        for i, w in enumerate(self.weights):
            if before_layer is not None:
                before_layer(i)
            h_in = h
            if i == 0 or self.q is None or self.q == 1.0:
                h = F.norm_dist(h, w, float("inf"))
            else:
                h = F.masked_inf_dist(h, w, self.q, seed=step_seed * 64 + i, mode=self.mask_mode)
            if after_layer is not None:
                after_layer(i, w)
            y, mean = h, None
            if i < self.num_layers - 1:
                h, mean = F.mean_shift(h, self.running_mean[i], self.momentum)
            else:
                h = h + self.bias.view(1, -1, 1)
            if trace is not None:
                trace.append((h_in.detach(), y.detach(), mean))
        return h.squeeze(-1)

    @torch.no_grad()
    def predict(self, x):
        """Evaluation forward of the pure l-inf net (q = 1): every layer without a mask, mean shift taken from
        the running means -- the value that `bounds()` brackets."""
        h = x.unsqueeze(-1).contiguous()
        for i, w in enumerate(self.weights):
            h = F.norm_dist(h, w, float("inf"))
            shift = self.running_mean[i].view(1, -1, 1) if i < self.num_layers - 1 else -self.bias.view(1, -1, 1)
            h = h - shift
        return h.squeeze(-1)

    @torch.no_grad()
    def bounds(self, lower, upper, means=None, before_layer=None):
        """Certification pass: interval bounds of the distances for inputs in [lower, upper].  `means` replaces the
        running means (a snapshot, for a caller that runs this pass beside a training forward that updates them);
        `before_layer(i)` as in `forward`."""
        means = self.running_mean if means is None else means
        lo, up = lower.unsqueeze(-1).contiguous(), upper.unsqueeze(-1).contiguous()
        for i, w in enumerate(self.weights):
            if before_layer is not None:
                before_layer(i)
            lo, up = F.bound_inf_dist(lo, up, w)
            shift = means[i].view(1, -1, 1) if i < self.num_layers - 1 else -self.bias.view(1, -1, 1)
            lo, up = lo - shift, up - shift
        return lo.squeeze(-1), up.squeeze(-1)


def margins(dist, targets, eps, lower=None, upper=None):
    """Logits and worst-case margins from class distances (ell_inf_models.py:45-50): without
    propagated bounds the 1-Lipschitz property gives dist -/+ eps."""
    lower = dist - eps if lower is None else lower
    upper = dist + eps if upper is None else upper
    logits, lo, up = -dist, -upper, -lower
    margin = up - torch.gather(lo, 1, targets.view(-1, 1))
    margin = margin.scatter(1, targets.view(-1, 1), 0)
    return logits, margin / (2 * eps)

"""Interval-bound versions of the dense head that follows the distance layers in the hybrid models
(core/models/bound_basic_module.py:11-103): ReLU / tanh, a linear layer, a convolution and the final linear
layer that returns worst-case margins against the target class.  Same constructor arguments, parameter names
(`weight`, `bias`), scaling (`w_scale = w_lr / sqrt(in_features)`, `b_scale = b_lr`) and
`(x, lower, upper)` protocol as the reference, so its checkpoints load.

These layers are matrix products, so they run on the library GEMMs behind torch.  The one difference in
formulation: the reference builds the whole (batch, classes, features) tensor `weight - weight[target]` for
the margin radius; here it is built for a bounded number of samples at a time (all of them for ten classes,
32 at a time for 1000 classes x 2048 features), so memory stays bounded for the many-class configurations.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as TF

from .layers import apply_if_not_none


class BoundReLU(nn.ReLU):
    def forward(self, x=None, lower=None, upper=None):      # monotone: bounds map to bounds
        return apply_if_not_none((x, lower, upper), TF.relu)


class BoundTanh(nn.Tanh):
    def forward(self, x=None, lower=None, upper=None):
        return apply_if_not_none((x, lower, upper), torch.tanh)


def _affine(inp, weight, bias, w_scale, b_scale):
    if bias is None:
        return torch.mm(inp, weight.t()) * w_scale
    return torch.addmm(bias, inp, weight.t(), alpha=w_scale, beta=b_scale)


class _ScaledLinear(nn.Linear):
    """nn.Linear with N(0, w_scale^2) weights, zero bias and the reference's run-time scaling."""

    def __init__(self, in_features, out_features, bias=True, w_scale=1.0, w_lr=1.0, b_lr=1.0):
        super().__init__(in_features, out_features, bias=bias)
        with torch.no_grad():
            self.weight.normal_().mul_(w_scale)
            if self.bias is not None:
                self.bias.zero_()
        self.w_scale = w_lr / math.sqrt(in_features)
        self.b_scale = b_lr

    def _center_radius(self, lower, upper):
        center = (lower + upper) * 0.5
        radius = (upper - lower) * 0.5
        return _affine(center, self.weight, self.bias, self.w_scale, self.b_scale), radius


class BoundLinear(_ScaledLinear):
    """core/models/bound_basic_module.py:27-47: W c + b -/+ |W| r for the box of centre c and radius r."""

    def forward(self, x=None, lower=None, upper=None):
        if x is not None:
            x = _affine(x, self.weight, self.bias, self.w_scale, self.b_scale)
        if lower is not None and upper is not None:
            z, radius = self._center_radius(lower, upper)
            spread = torch.mm(radius, self.weight.abs().t()) * self.w_scale
            lower, upper = z - spread, z + spread
        return x, lower, upper


class BoundConv2d(nn.Conv2d):
    """core/models/bound_basic_module.py:50-76: the convolution counterpart of BoundLinear, with
    `w_scale = w_lr / sqrt(in_channels * kernel_size^2)`; the box is propagated as centre and radius
    (radius through |W|, no bias)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1, bias=True,
                 w_scale=1.0, w_lr=1.0, b_lr=1.0):
        super().__init__(in_channels, out_channels, kernel_size, stride=stride, padding=padding, dilation=dilation,
                         groups=groups, bias=bias)
        with torch.no_grad():
            self.weight.normal_().mul_(w_scale)
            if self.bias is not None:
                self.bias.zero_()
        self.w_scale = w_lr / math.sqrt(in_channels * kernel_size * kernel_size)
        self.b_scale = b_lr

    def _conv(self, inp, weight, with_bias):
        bias = self.bias * self.b_scale if with_bias and self.bias is not None else None
        return TF.conv2d(inp, weight, bias, stride=self.stride, padding=self.padding, dilation=self.dilation,
                         groups=self.groups)

    def forward(self, x=None, lower=None, upper=None):
        if x is not None:
            x = self._conv(x, self.weight * self.w_scale, True)
        if lower is not None and upper is not None:
            half = self.w_scale / 2
            z = self._conv(lower + upper, self.weight * half, True)
            spread = self._conv(upper - lower, self.weight.abs() * half, False)
            lower, upper = z - spread, z + spread
        return x, lower, upper


class BoundFinalLinear(_ScaledLinear):
    """core/models/bound_basic_module.py:79-103.  Without bounds or targets: the logits.  With both:
    `(logits, res)`, `res[b, j]` = upper bound over the box of `logit_j - logit_target(b)` (0 at j = target)."""

    max_diff_elements = 1 << 26  # largest (samples, classes, features) difference tensor formed at once (256 MiB)

    def forward(self, x=None, lower=None, upper=None, targets=None):
        if x is not None:
            x = _affine(x, self.weight, self.bias, self.w_scale, self.b_scale)
            if lower is None or upper is None or targets is None:
                return x
        res = None
        if lower is not None and upper is not None and targets is not None:
            z, radius = self._center_radius(lower, upper)
            z = z - torch.gather(z, 1, targets.unsqueeze(1))
            res = z + self._margin_radius(radius, targets) * self.w_scale
        return x, res

    def _margin_radius(self, radius, targets):
        """sum_i |W[j, i] - W[target_b, i]| radius[b, i] for every sample b and class j, in chunks of samples
        sized by `max_diff_elements`; no data-dependent shapes, hence no host synchronisation."""
        w = self.weight
        chunk = max(1, self.max_diff_elements // (w.size(0) * w.size(1)))
        pieces = []
        for start in range(0, radius.size(0), chunk):
            t = targets[start:start + chunk]
            diff = (w.unsqueeze(0) - w.index_select(0, t).unsqueeze(1)).abs()      # (chunk, classes, features)
            pieces.append(torch.bmm(diff, radius[start:start + chunk].unsqueeze(-1)).squeeze(-1))
        return pieces[0] if len(pieces) == 1 else torch.cat(pieces)

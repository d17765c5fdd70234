"""Distance layers on top of `sortnet_amd.functional`: the callers of the hot path.

Same construction arguments, `(x, lower, upper) -> (x, lower, upper)` protocol (None = absent) and
mode selection as the reference's core/models/norm_dist.py (`NormDistBase`, `NormDist`, `NormDistConv`)
and core/models/bound_basic_module.py (`MeanShiftDropout`, `BoundSequential`):

* training with a keep probability registered on some layer: kept-channel index lists per 32-sample
  sub-batch, `norm_dist_dropout` on the compacted input, index-aware mean shift
  (core/models/norm_dist.py:52-85);
* evaluation with keep probabilities registered: `sort_neuron` for the value and `bound_sort_neuron`
  for the bounds (:86-91);
* no keep probability anywhere: `norm_dist` / `bound_inf_dist` (:92-97).

Differences: the index lists come from the library's device-side sampler (stateless counter RNG, no
`.item()` synchronisation with the device; `set_mask_seed` makes a run reproducible), and the registry
that lets neighbouring layers share a mask is an explicit object (`DropoutRegistry`, one default
instance) instead of class attributes, so two models can live in one process.
"""
import math
from collections.abc import Iterable

import torch
import torch.nn as nn
import torch.nn.functional as TF

from . import ext
from . import functional as F

SUB_BATCH = 32   # samples that share one index list (core/cuda/inf_dist_cuda.cu:8)


def apply_if_not_none(paras, func):
    return [None if x is None else func(x) for x in paras]


class DropoutRegistry:
    """What the reference keeps in NormDistBase.dropout_list / dropout_buffer / tag
    (core/models/norm_dist.py:21-23): which layers drop which share of their inputs, the mask a
    layer sampled for the inputs of its successor, and the seed counter of the sampler."""

    def __init__(self, seed=0):
        self.entries = {}      # tag -> (inputs per group, outputs per group, keep probability)
        self.buffer = None     # (tag of the consumer, w_index_ci)
        self.next_tag = 0
        self.seed = seed
        self.draws = 0
        self.overlap_sampler = True
        self._side_streams = {}

    def new_tag(self):
        self.next_tag += 1
        return self.next_tag

    def sample(self, sub_batches, groups, channels, q, device):
        """Ascending kept-channel lists (sub_batches, groups, count), count ~ Binomial(channels, q).
        The lists depend on nothing but the seed, and the sampler keeps only a few compute units busy, so it
        is queued on a second stream (default priority) and overlaps the kernels already queued on the
        caller's stream; the caller's stream waits for it before going on."""
        self.draws += 1
        seed = (self.seed * 1000003 + self.draws) & 0xFFFFFFFF
        count = ext.mask_count(seed, channels, q)
        device = torch.device(device)
        if device.type != "cuda" or not self.overlap_sampler:
            return ext.sample_index_lists(seed, sub_batches, groups, channels, count, device)
        main = torch.cuda.current_stream(device)
        side = self._side_streams.get(device)
        if side is None:
            side = self._side_streams[device] = torch.cuda.Stream(device=device)
        with torch.cuda.stream(side):
            lists = ext.sample_index_lists(seed, sub_batches, groups, channels, count, device)
        main.wait_stream(side)
        lists.record_stream(main)
        return lists


DEFAULT_REGISTRY = DropoutRegistry()


def set_mask_seed(seed, registry=DEFAULT_REGISTRY):
    registry.seed, registry.draws = seed, 0


class MeanShiftDropout(nn.Module):
    """core/models/bound_basic_module.py:106-157."""

    def __init__(self, out_channels, momentum=0.1, affine=True):
        super().__init__()
        self.out_channels, self.momentum = out_channels, momentum
        self.register_buffer("running_mean", torch.zeros(out_channels))
        self.bias = nn.Parameter(torch.zeros(out_channels)) if affine else None

    def forward(self, x=None, lower=None, upper=None, index=None):
        if self.training:
            assert x is not None, "Currently not supported"
            if self.bias is None and lower is None and upper is None:
                # fused kernels: mean, running-mean update and subtraction (own backward)
                if index is None:
                    x, _ = F.mean_shift(x.contiguous(), self.running_mean, self.momentum)
                else:
                    x, _ = F.mean_shift_index(x, index.to(torch.int32).contiguous(), self.out_channels,
                                              self.running_mean, self.momentum)
                return x, lower, upper
            # bounds alongside x, or an affine bias: the batch mean of x, inside the graph, is subtracted from
            # all three (core/models/bound_basic_module.py:125-157)
            index = None if index is None else index.long()
            mean = self._batch_mean(x, index)
            with torch.no_grad():
                self.running_mean.mul_(1 - self.momentum).add_(mean, alpha=self.momentum)
        else:
            mean = self.running_mean
        if self.bias is not None:
            mean = mean - self.bias
        if index is not None:
            index = index.long()
            rows = torch.div(torch.arange(x.size(0), device=x.device), SUB_BATCH, rounding_mode="trunc")
            per_row = mean.view(1, index.size(-2), -1).expand(x.size(0), -1, -1)
            mean_b = torch.gather(per_row, -1, index[rows]).reshape(x.size(0), -1).unsqueeze(-1)
            return tuple(apply_if_not_none((x, lower, upper), lambda z: z - mean_b))
        return tuple(apply_if_not_none((x, lower, upper), lambda z: _shift(z, mean, -1.0)))

    def _batch_mean(self, x, index):
        if index is None:
            return x.mean(dim=(0, 2))
        # every sub-batch contributes its samples to the channels of its own index list
        b, groups = x.size(0), index.size(-2)
        pad = (-b) % SUB_BATCH
        xp = torch.cat((x, x.new_zeros(pad, x.size(1), x.size(2)))) if pad else x
        sums = xp.view(index.size(0), SUB_BATCH, groups, -1, x.size(-1)).transpose(0, 2).sum(dim=(1, -1))
        flat = index.transpose(0, 1).reshape(groups, -1)
        total = x.new_zeros(groups, self.out_channels // groups).scatter_add(1, flat, sums.reshape(groups, -1))
        cnt = x.new_full(index.transpose(0, 1).shape, float(SUB_BATCH))
        if pad:
            cnt[:, -1] = SUB_BATCH - pad
        seen = x.new_full((groups, self.out_channels // groups), 1e-10).scatter_add(1, flat, cnt.reshape(groups, -1))
        return (total / (seen * x.size(-1))).view(-1)


def _shift(z, vec, sign):
    """z + sign * vec[channel].  The kernel form has no backward, so it only serves tensors outside a graph
    (the attack differentiates an evaluation-mode stack with respect to its input, attack.py:26-29)."""
    if torch.is_grad_enabled() and (z.requires_grad or vec.requires_grad):
        return z + sign * vec.view(1, -1, 1)
    out = torch.empty_like(z)
    ext.channel_shift(z.contiguous(), vec.contiguous(), sign, out)
    return out


class NormDistBase(nn.Module):
    """core/models/norm_dist.py:20-104."""

    def __init__(self, in_features, out_features, p=float("inf"), groups=1, bias=True, std=1.0, mean_shift=True,
                 dropout=None, registry=None):
        super().__init__()
        assert in_features % groups == 0 and out_features % groups == 0
        self.weight = nn.Parameter(torch.randn(out_features, in_features // groups) * std)
        self.groups, self.p = groups, p
        self.bias = nn.Parameter(torch.zeros(out_features)) if bias else None
        self.mean_shift = MeanShiftDropout(out_features, affine=False) if mean_shift else None
        self.registry = registry if registry is not None else DEFAULT_REGISTRY
        self.tag = self.registry.new_tag()
        self.dropout = dropout
        if dropout is not None:
            self.registry.entries[self.tag] = (in_features // groups, out_features // groups, dropout)

    def forward(self, x=None, lower=None, upper=None):
        reg = self.registry
        index_out, bias = None, self.bias
        if reg.entries:
            assert x is not None
            grad = torch.is_grad_enabled() and (x.requires_grad or self.weight.requires_grad)
            assert (grad and self.training) or math.isinf(self.p)
            if grad and self.training:
                x, index_out, bias = self._forward_index_lists(x)
            else:
                x = F.sort_neuron(x, self.weight, self.groups, q=self.dropout, tag=self.tag)
                if lower is not None and upper is not None:
                    lower, upper = F.bound_sort_neuron(lower, upper, self.weight, self.groups, q=self.dropout,
                                                       tag=self.tag)
        else:
            if x is not None:
                x = F.norm_dist(x, self.weight, self.p, self.groups, tag=self.tag)
            if lower is not None and upper is not None:
                assert math.isinf(self.p)
                lower, upper = F.bound_inf_dist(lower, upper, self.weight, self.groups, tag=self.tag)
        if self.mean_shift is not None:
            x, lower, upper = self.mean_shift(x, lower, upper, index=index_out)
        if bias is not None:
            x, lower, upper = apply_if_not_none((x, lower, upper), lambda z: z + bias.unsqueeze(-1))
        return x, lower, upper

    def _forward_index_lists(self, x):
        """Training path with kept-channel lists (core/models/norm_dist.py:55-85)."""
        reg, dev = self.registry, x.device
        sub_batches = (x.size(0) - 1) // SUB_BATCH + 1
        rows = torch.div(torch.arange(x.size(0), device=dev), SUB_BATCH, rounding_mode="trunc")
        dim_out = self.weight.size(0) // self.groups
        index_in = None
        if self.tag in reg.entries and self.dropout != 1.0:
            dim_in, dim_out, q = reg.entries[self.tag]
            if reg.buffer is not None and reg.buffer[0] == self.tag:
                index_in = reg.buffer[1]          # the predecessor already produced compacted outputs
            else:
                index_in = reg.sample(sub_batches, self.groups, dim_in, q, dev)
                xg = x.view(x.size(0), self.groups, -1, x.size(-1))
                gather = index_in[rows].unsqueeze(-1).long().expand(-1, -1, -1, x.size(-1))
                x = torch.gather(xg, 2, gather).reshape(x.size(0), -1, x.size(-1))
        index_out, bias = None, self.bias
        nxt = reg.entries.get(self.tag + 1)
        if nxt is not None and nxt[0] == dim_out and nxt[2] != 1.0:
            index_out = reg.sample(sub_batches, self.groups, dim_out, nxt[2], dev)
            reg.buffer = (self.tag + 1, index_out)
            if self.bias is not None:
                per_row = self.bias.view(1, self.groups, -1).expand(x.size(0), -1, -1)
                bias = torch.gather(per_row, -1, index_out[rows].long()).reshape(x.size(0), -1)
        y = F.norm_dist_dropout(x.contiguous(), self.weight, index_in, index_out, self.p, self.groups, tag=self.tag)
        return y, index_out, bias


class NormDist(NormDistBase):
    """Fully connected distance layer on (B, features) tensors (core/models/norm_dist.py:107-127)."""

    def __init__(self, in_features, out_features, groups=1, bias=True, identity_val=None, **kwargs):
        super().__init__(in_features, out_features, groups=groups, bias=bias, **kwargs)
        self.in_features, self.out_features = in_features, out_features
        if identity_val is not None and in_features <= out_features:
            with torch.no_grad():
                cols = torch.arange(out_features) % (in_features // groups)
                self.weight[torch.arange(out_features), cols] = -identity_val

    def forward(self, x=None, lower=None, upper=None):
        paras = apply_if_not_none((x, lower, upper), lambda z: z.unsqueeze(-1))
        paras = super().forward(*paras)
        return tuple(apply_if_not_none(paras, lambda z: z.squeeze(-1)))


class NormDistConv(NormDistBase):
    """Convolutional distance layer through unfold (core/models/norm_dist.py:130-164)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, identity_val=None, **kwargs):
        ks = tuple(kernel_size) if isinstance(kernel_size, Iterable) else (kernel_size, kernel_size)
        assert in_channels % groups == 0
        super().__init__(in_channels * ks[0] * ks[1], out_channels, groups=groups, bias=bias, **kwargs)
        self.kernel_size, self.stride, self.padding, self.dilation = ks, stride, padding, dilation
        if identity_val is not None and in_channels <= out_channels:
            with torch.no_grad():
                wv = self.weight.view(out_channels, -1, *ks)
                for i in range(out_channels):
                    wv[i, i % (in_channels // groups), ks[0] // 2, ks[1] // 2] = -identity_val

    def forward(self, x=None, lower=None, upper=None):
        ref = x if x is not None else lower
        h, w = ref.size(2), ref.size(3)
        unfold = lambda z: TF.unfold(z, self.kernel_size, self.dilation, self.padding, self.stride).contiguous()
        paras = super().forward(*apply_if_not_none((x, lower, upper), unfold))
        h, w = [(s + 2 * self.padding - self.dilation * (k - 1) - 1) // self.stride + 1
                for s, k in zip((h, w), self.kernel_size)]
        return tuple(apply_if_not_none(paras, lambda z: z.reshape(z.size(0), -1, h, w)))


class BoundSequential(nn.Sequential):
    """core/models/bound_basic_module.py:163-167."""

    def forward(self, paras):
        for module in self:
            paras = module(*paras)
        return paras

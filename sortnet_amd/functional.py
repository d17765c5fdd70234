"""Functional / autograd front-end of the distance-neuron kernels.

Public names, positional order, defaults, return shapes and dtypes follow the reference's
core/norm_dist.py (file:line cited per symbol) so that its layers (core/models/norm_dist.py)
run unmodified on top of this module.  Inputs are 3-D (B, C, HW) fp32 tensors on the GPU,
weight is (CO, CI / groups); outputs are fp32 on the input's device, positions are int32.

Every function dispatches to the HIP kernels through `sortnet_amd.ext`.  `use_custom_cuda_func=False`
selects, as in the reference, a formulation in plain torch ops on the tensors' own device (differentiable
by autograd, formed for a bounded number of output channels at a time); it is a second, independent
statement of the same values and nothing in this library calls it on its own.
"""
import math

import torch

from . import ext as _C

__all__ = [
    "NormDistF", "NormDistDropoutF", "SortNeuronF", "BoundInfDistF", "MaskedInfDistF",
    "norm_dist", "norm_dist_dropout", "sort_neuron", "bound_sort_neuron", "bound_inf_dist", "masked_inf_dist",
    "MeanShiftF", "mean_shift", "MeanShiftIndexF", "mean_shift_index",
]


def _new_out(x, channels):
    return torch.empty(x.size(0), channels, x.size(2), device=x.device, dtype=torch.float32)


def _want_grad(*tensors):
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


# ---- use_custom_cuda_func=False: the reference's closed forms in torch ops ---------------------------------------
# The reference forms the whole (B, G, CO/G, CI/G, HW) tensor of differences at once (53.7 GB at B=512,
# CO=CI=5120); here the output channels go by in blocks whose differences stay below _TORCH_BLOCK_BYTES.
_TORCH_BLOCK_BYTES = 256 << 20


def _blocks_of_differences(inputs, weight, groups):
    """Yields, group by group and block by block of output channels, the differences
    d[k][b, m, n, hw] = inputs[k][b, g, n, hw] - weight[g, m, n] for every tensor of `inputs`, in the order in
    which the outputs are laid out ((B, G * CO/G, HW), group-major)."""
    B, C, HW = inputs[0].shape
    cig = C // groups
    cog = weight.size(0) // groups
    w = weight.view(groups, cog, cig)
    step = max(1, _TORCH_BLOCK_BYTES // max(1, 4 * len(inputs) * B * cig * HW))
    for g in range(groups):
        xs = [t[:, g * cig:(g + 1) * cig, :].unsqueeze(1) for t in inputs]        # (B, 1, cig, HW)
        for m0 in range(0, cog, step):
            wb = w[g, m0:m0 + step].unsqueeze(0).unsqueeze(-1)                    # (1, mc, cig, 1)
            yield [x - wb for x in xs]


def _torch_norm_dist(x, weight, p, groups):
    """core/norm_dist.py:181-185: the l-p norm of the differences, scaled by their largest magnitude (which is
    held constant under differentiation) so that large p neither overflows nor underflows."""
    out = []
    for (d,) in _blocks_of_differences([x], weight, groups):
        with torch.no_grad():
            scale = d.abs().amax(dim=2, keepdim=True)
        out.append((torch.linalg.vector_norm(d / scale, ord=p, dim=2, keepdim=True) * scale).squeeze(2))
    return torch.cat(out, dim=1)


def _torch_sort_neuron(x, weight, groups, q, truncate):
    """core/norm_dist.py:226-230: the `truncate` largest magnitudes, weighted q (1 - q)^j from the largest down and
    normalised by 1 - (1 - q)^truncate (no 1e-10 floor in this form)."""
    coef = ((1 - q) ** torch.arange(truncate, device=x.device, dtype=x.dtype) * q).view(1, 1, truncate, 1)
    out = []
    for (d,) in _blocks_of_differences([x], weight, groups):
        top = torch.topk(d.abs(), k=truncate, dim=2)[0]                            # (B, mc, truncate, HW), descending
        out.append((top * coef).sum(dim=2))
    return torch.cat(out, dim=1) / (1 - (1 - q) ** truncate)


def _torch_bound_inf_dist(x_lower, x_upper, weight, groups):
    """core/norm_dist.py:251-259: per input the two ends w - l and u - w; the upper result is the largest of their
    maxima and the lower result minus the smallest of their minima, both floored at 1e-10 (this form does not
    repair inverted intervals)."""
    lo, up = [], []
    for dl, du in _blocks_of_differences([x_lower, x_upper], weight, groups):
        t1, t2 = -dl, du
        up.append(torch.maximum(t1, t2).clamp(min=1e-10).amax(dim=2))
        lo.append((-torch.minimum(t1, t2).clamp(max=-1e-10)).amax(dim=2))
    return torch.cat(lo, dim=1), torch.cat(up, dim=1)


def _torch_norm_dist_dropout(x, weight, w_index_ci, w_index_co, p, groups):
    """core/norm_dist.py:195-213 without the kernels: each 32-sample sub-batch meets the sub-matrix of the weight
    that its two index lists select (a missing list keeps everything)."""
    cog, cig = weight.size(0) // groups, weight.size(1)
    w = weight.view(groups, cog, cig)
    out = []
    for s, b0 in enumerate(range(0, x.size(0), 32)):
        rows = []
        for g in range(groups):
            wg = w[g]
            if w_index_co is not None:
                wg = wg.index_select(0, w_index_co[s, g].long())
            if w_index_ci is not None:
                wg = wg.index_select(1, w_index_ci[s, g].long())
            rows.append(wg)
        out.append(_torch_norm_dist(x[b0:b0 + 32], torch.cat(rows, dim=0), p, groups))
    return torch.cat(out, dim=0)


class NormDistF(torch.autograd.Function):
    """l-p (finite p) or l-inf (p = inf) distance layer.  Mirrors core/norm_dist.py:6-51."""

    @staticmethod
    def forward(ctx, x, weight, group, p, need_grad, tag):
        assert weight.size(1) * group == x.size(1)
        y = _new_out(x, weight.size(0))
        ctx.group, ctx.p, ctx.tag = group, p, tag
        if math.isinf(p):
            if need_grad:
                pos = torch.empty_like(y, dtype=torch.int)
                _C.inf_dist_forward(x, weight, y, pos, group)
                ctx.save_for_backward(x, weight, pos)
            else:
                _C.inf_dist_forward_nograd(x, weight, y, group)
        elif p > 0:
            _C.norm_dist_forward(x, weight, y, group, p)
            ctx.save_for_backward(x, weight, y)
        else:
            raise NotImplementedError
        return y

    @staticmethod
    def backward(ctx, grad_output):
        grad_output = grad_output.contiguous()
        want_x, want_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        grad_weight = None
        if math.isinf(ctx.p):
            x, weight, pos = ctx.saved_tensors
            grad_input = torch.empty_like(x)
            if want_w:
                grad_weight = torch.empty_like(weight)
                _C.inf_dist_backward_input_weight(grad_output, pos, grad_input, grad_weight, ctx.group)
            elif want_x:
                _C.inf_dist_backward_input(grad_output, pos, grad_input, ctx.group)
        else:
            x, weight, y = ctx.saved_tensors
            grad_input = torch.empty_like(x)
            if want_w:
                grad_weight = torch.empty_like(weight)
                _C.norm_dist_backward_input_weight(grad_output, x, weight, y, grad_input, grad_weight,
                                                   ctx.group, ctx.p)
            elif want_x:
                _C.norm_dist_backward_input(grad_output, x, weight, y, grad_input, ctx.group, ctx.p)
        return (grad_input if want_x else None), grad_weight, None, None, None, None


class NormDistDropoutF(torch.autograd.Function):
    """Distance layer on index-list sub-matrices of the weight, one list per 32-sample sub-batch.
    Mirrors core/norm_dist.py:54-99."""

    @staticmethod
    def forward(ctx, x, weight, w_index_ci, w_index_co, group, p, tag):
        channels = weight.size(0) if w_index_co is None else w_index_co.size(-1) * group
        assert weight.size(1) * group == x.size(1) or w_index_ci.size(-1) * group == x.size(1)
        y = _new_out(x, channels)
        ctx.group, ctx.p, ctx.tag = group, p, tag
        if math.isinf(p):
            pos = torch.empty_like(y, dtype=torch.int)
            _C.inf_dist_forward(x, weight, y, pos, group, w_index_ci, w_index_co)
            ctx.save_for_backward(x, weight, pos, w_index_ci, w_index_co)
        elif p > 0:
            _C.norm_dist_forward(x, weight, y, group, p, w_index_ci, w_index_co)
            ctx.save_for_backward(x, weight, y, w_index_ci, w_index_co)
        else:
            raise NotImplementedError
        return y

    @staticmethod
    def backward(ctx, grad_output):
        grad_output = grad_output.contiguous()
        want_x, want_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        grad_weight = None
        if math.isinf(ctx.p):
            x, weight, pos, w_index_ci, w_index_co = ctx.saved_tensors
            grad_input = torch.empty_like(x)
            if want_w:
                grad_weight = torch.empty_like(weight)
                _C.inf_dist_backward_input_weight(grad_output, pos, grad_input, grad_weight, ctx.group,
                                                  w_index_ci, w_index_co)
            elif want_x:
                _C.inf_dist_backward_input(grad_output, pos, grad_input, ctx.group)
        else:
            x, weight, y, w_index_ci, w_index_co = ctx.saved_tensors
            grad_input = torch.empty_like(x)
            if want_w:
                grad_weight = torch.empty_like(weight)
                _C.norm_dist_backward_input_weight(grad_output, x, weight, y, grad_input, grad_weight,
                                                   ctx.group, ctx.p, w_index_ci, w_index_co)
            elif want_x:
                _C.norm_dist_backward_input(grad_output, x, weight, y, grad_input, ctx.group, ctx.p,
                                            w_index_ci, w_index_co)
        return (grad_input if want_x else None), grad_weight, None, None, None, None, None


class SortNeuronF(torch.autograd.Function):
    """Geometric-weighted sum of the top-`truncate` values of |x - w|.  Mirrors core/norm_dist.py:102-133."""

    @staticmethod
    def forward(ctx, x, weight, group, q, truncate, need_grad, tag):
        assert weight.size(1) * group == x.size(1)
        y = _new_out(x, weight.size(0))
        ctx.group, ctx.q, ctx.truncate, ctx.tag = group, q, truncate, tag
        if need_grad:
            pos = torch.empty(truncate, x.size(0), weight.size(0), x.size(2), device=x.device, dtype=torch.int)
            _C.sort_neuron_forward(x, weight, y, pos, group, q, truncate)
            ctx.save_for_backward(x, weight, pos)
        else:
            _C.sort_neuron_forward_nograd(x, weight, y, group, q, truncate)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x, weight, pos = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        want_x, want_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        grad_input = torch.empty_like(x)
        grad_weight = None
        if want_w:
            grad_weight = torch.empty_like(weight)
            _C.sort_neuron_backward_input_weight(grad_output, pos, grad_input, grad_weight, ctx.group, ctx.q,
                                                 ctx.truncate)
        elif want_x:
            _C.sort_neuron_backward_input(grad_output, pos, grad_input, ctx.group, ctx.q, ctx.truncate)
        return (grad_input if want_x else None), grad_weight, None, None, None, None, None


class BoundInfDistF(torch.autograd.Function):
    """Interval bounds through the l-inf layer, forward and backward.  Mirrors core/norm_dist.py:136-173."""

    @staticmethod
    def forward(ctx, x_lower, x_upper, weight, group, need_grad, tag):
        assert x_lower.size() == x_upper.size()
        assert weight.size(1) * group == x_lower.size(1)
        y_lower = _new_out(x_lower, weight.size(0))
        y_upper = torch.empty_like(y_lower)
        ctx.group, ctx.tag = group, tag
        if need_grad:
            pos_lower = torch.empty_like(y_lower, dtype=torch.int)
            pos_upper = torch.empty_like(pos_lower)
            _C.bound_inf_dist_forward(x_lower, x_upper, weight, y_lower, y_upper, pos_lower, pos_upper, group)
            ctx.save_for_backward(x_lower, x_upper, weight, pos_lower, pos_upper)
        else:
            _C.bound_inf_dist_forward_nograd(x_lower, x_upper, weight, y_lower, y_upper, group)
        return y_lower, y_upper

    @staticmethod
    def backward(ctx, grad_y_lower, grad_y_upper):
        grad_y_lower = grad_y_lower.contiguous()
        grad_y_upper = grad_y_upper.contiguous()
        x_lower, x_upper, weight, pos_lower, pos_upper = ctx.saved_tensors
        want_l, want_u, want_w = ctx.needs_input_grad[:3]
        grad_x_lower = torch.zeros_like(x_lower)
        grad_x_upper = torch.zeros_like(x_upper)
        grad_weight = None
        if want_w:
            grad_weight = torch.zeros_like(weight)
            _C.bound_inf_dist_backward_input_weight(grad_y_lower, grad_y_upper, pos_lower, pos_upper,
                                                    grad_x_lower, grad_x_upper, grad_weight, ctx.group)
        elif want_l and want_u:
            _C.bound_inf_dist_backward_input(grad_y_lower, grad_y_upper, pos_lower, pos_upper,
                                             grad_x_lower, grad_x_upper, ctx.group)
        return (grad_x_lower if want_l else None), (grad_x_upper if want_u else None), grad_weight, None, None, None


class MaskedInfDistF(torch.autograd.Function):
    """SortNet's training neuron as one fused op: max over a Bernoulli(q)-kept subset of |x - w|,
    the keep decisions drawn on the GPU from a stateless counter RNG of (seed, b, m, n).
    The reference builds the same kind of subset on the host (core/models/norm_dist.py:14-17) and
    feeds index lists to NormDistDropoutF; the backward here is the l-inf scatter through the
    saved arg-max index, identical to NormDistF's (core/norm_dist.py:29-39)."""

    @staticmethod
    def forward(ctx, x, weight, group, q, seed, mode, need_grad, tag):
        assert weight.size(1) * group == x.size(1)
        y = _new_out(x, weight.size(0))
        ctx.group, ctx.tag = group, tag
        if need_grad:
            pos = torch.empty_like(y, dtype=torch.int)
            _C.masked_inf_dist_forward(x, weight, y, pos, group, q, seed, mode)
            ctx.save_for_backward(x, weight, pos)
        else:
            _C.masked_inf_dist_forward(x, weight, y, None, group, q, seed, mode)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x, weight, pos = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        want_x, want_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        grad_input = torch.empty_like(x)
        grad_weight = None
        if want_w:
            grad_weight = torch.empty_like(weight)
            _C.inf_dist_backward_input_weight(grad_output, pos, grad_input, grad_weight, ctx.group)
        elif want_x:
            _C.inf_dist_backward_input(grad_output, pos, grad_input, ctx.group)
        return (grad_input if want_x else None), grad_weight, None, None, None, None, None, None


class MeanShiftF(torch.autograd.Function):
    """y = x - mean_{b,hw}(x) with the mean inside the graph, plus the running-mean update the
    reference's MeanShiftDropout does under no_grad (core/models/bound_basic_module.py:123-157, the
    form without an index list).  The backward of the centring is the centring of the gradient."""

    @staticmethod
    def forward(ctx, x, running_mean, momentum):
        x = x.contiguous()
        y = torch.empty_like(x)
        mean = torch.empty(x.size(1), device=x.device, dtype=torch.float32)
        _C.mean_shift_forward(x, mean, running_mean, momentum, y)
        ctx.mark_non_differentiable(mean)
        return y, mean

    @staticmethod
    def backward(ctx, grad_y, _grad_mean):
        grad_y = grad_y.contiguous()
        grad_x = torch.empty_like(grad_y)
        scratch = torch.empty(grad_y.size(1), device=grad_y.device, dtype=torch.float32)
        _C.mean_shift_forward(grad_y, scratch, None, 0.0, grad_x)
        return grad_x, None, None


class MeanShiftIndexF(torch.autograd.Function):
    """MeanShiftF when every 32-sample sub-batch keeps its own channels (`index`, shape (S, G, cnt)):
    the mean of a channel runs over the sub-batches that kept it
    (core/models/bound_basic_module.py:125-137,146-153).  The backward is the same centring of the gradient."""

    @staticmethod
    def forward(ctx, x, index, channels, running_mean, momentum):
        x = x.contiguous()
        y = torch.empty_like(x)
        mean = torch.empty(channels, device=x.device, dtype=torch.float32)
        _C.mean_shift_index_forward(x, index, channels // index.size(-2), mean, running_mean, momentum, y)
        ctx.save_for_backward(index)
        ctx.channels = channels
        ctx.mark_non_differentiable(mean)
        return y, mean

    @staticmethod
    def backward(ctx, grad_y, _grad_mean):
        index, = ctx.saved_tensors
        grad_y = grad_y.contiguous()
        grad_x = torch.empty_like(grad_y)
        scratch = torch.empty(ctx.channels, device=grad_y.device, dtype=torch.float32)
        _C.mean_shift_index_forward(grad_y, index, ctx.channels // index.size(-2), scratch, None, 0.0, grad_x)
        return grad_x, None, None, None, None


def mean_shift_index(x, index, channels, running_mean=None, momentum=0.1):
    """Training-mode mean shift of a compacted (B, G * cnt, HW) tensor; `channels` counts all channels of all
    groups.  Returns (x - mean[index], mean) and updates `running_mean` in place when given."""
    return MeanShiftIndexF.apply(x, index, channels, running_mean, momentum)


def mean_shift(x, running_mean=None, momentum=0.1):
    """Training-mode mean shift of a (B, C, HW) tensor; returns (x - mean, mean) and updates
    `running_mean` in place when given."""
    return MeanShiftF.apply(x, running_mean, momentum)


def norm_dist(input, weight, p, groups=1, use_custom_cuda_func=True, tag=None):
    """core/norm_dist.py:176-186."""
    if not use_custom_cuda_func:
        return _torch_norm_dist(input, weight, p, groups)
    return NormDistF.apply(input, weight, groups, p, _want_grad(input, weight), tag)


def norm_dist_dropout(input, weight, w_index_ci, w_index_co, p, groups=1, use_custom_cuda_func=True, tag=None):
    """core/norm_dist.py:191-214.  `input` is already compacted to the kept channels; `weight` is the
    full tensor; the same index list serves the 32 samples of a sub-batch."""
    if not use_custom_cuda_func:
        return _torch_norm_dist_dropout(input, weight, w_index_ci, w_index_co, p, groups)
    return NormDistDropoutF.apply(input, weight, w_index_ci, w_index_co, groups, p, tag)


def sort_neuron(input, weight, groups=1, q=0.5, truncate=10, use_custom_cuda_func=True, tag=None):
    """core/norm_dist.py:217-231."""
    truncate = min(weight.size(-1), truncate)
    if q is None or q == 1.0 or truncate == 1:
        return norm_dist(input, weight, float("inf"), groups, tag=tag)
    if not use_custom_cuda_func:
        return _torch_sort_neuron(input, weight, groups, q, truncate)
    return SortNeuronF.apply(input, weight, groups, q, truncate, _want_grad(input, weight), tag)


def bound_sort_neuron(x_lower, x_upper, weight, groups=1, q=0.5, truncate=10, tag=None):
    """core/norm_dist.py:234-243.  Forward only, as in the reference."""
    truncate = min(weight.size(-1), truncate)
    if q is None or q == 1.0 or truncate == 1:
        return bound_inf_dist(x_lower, x_upper, weight, groups, tag=tag)
    assert not _want_grad(x_lower, x_upper, weight)
    y_lower = _new_out(x_lower, weight.size(0))
    y_upper = torch.empty_like(y_lower)
    _C.bound_sort_neuron_forward(x_lower, x_upper, weight, y_lower, y_upper, groups, q, truncate)
    return y_lower, y_upper


def bound_inf_dist(x_lower, x_upper, weight, groups=1, use_custom_cuda_func=True, tag=None):
    """core/norm_dist.py:246-260."""
    if not use_custom_cuda_func:
        return _torch_bound_inf_dist(x_lower, x_upper, weight, groups)
    return BoundInfDistF.apply(x_lower, x_upper, weight, groups, _want_grad(x_lower, x_upper, weight), tag)


def masked_inf_dist(input, weight, q, seed, groups=1, mode=_C.MASK_TERM, tag=None):
    """Masked order-statistic neuron (see MaskedInfDistF).  `mode` is ext.MASK_TERM (independent
    draw per term) or ext.MASK_FACTORED (keep = keep_x(b, n) & keep_w(m, n))."""
    if q is None or q == 1.0:
        return norm_dist(input, weight, float("inf"), groups, tag=tag)
    return MaskedInfDistF.apply(input, weight, groups, q, seed, mode, _want_grad(input, weight), tag)

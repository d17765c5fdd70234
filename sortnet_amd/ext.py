"""Tensor-level mirror of the reference's compiled extension module `norm_dist_cuda`
(core/cuda/norm_dist.cpp:294-317): same function names, argument order and in-place output
convention, so `import sortnet_amd.ext as _C` can stand in for `import norm_dist_cuda as _C`.

Like the reference (norm_dist.cpp:9-12) every tensor must live on the GPU and be contiguous;
sizes are derived from the tensors exactly as the reference derives them.  Work is queued on
torch's current stream of the tensors' device.
"""
import torch

from . import _lib

MASK_TERM = 0
MASK_FACTORED = 1


def _chk(t, name, dtype=torch.float32):
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if t.dtype != dtype:
        raise RuntimeError("%s must have dtype %s" % (name, dtype))
    return t.data_ptr()


def _opt(t, name):
    return None if t is None else _chk(t, name, torch.int32)


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _run(name, ref, *args):
    with torch.cuda.device(ref.device):
        _lib.call(name, *args, _stream(ref))


def norm_dist_forward(input, weight, output, G, p, w_index_ci=None, w_index_co=None):
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _run("sd_norm_dist_forward", input, _chk(input, "input"), _chk(weight, "weight"), B, CO, CI, G, HW,
         _chk(output, "output"), p, _opt(w_index_ci, "w_index_ci"), _opt(w_index_co, "w_index_co"),
         weight.size(0), weight.size(1) * G)


def norm_dist_forward_with_max(input, weight, max_output, output, G, p, w_index_ci=None, w_index_co=None):
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _run("sd_norm_dist_forward_with_max", input, _chk(input, "input"), _chk(weight, "weight"),
         _chk(max_output, "max_output"), B, CO, CI, G, HW, _chk(output, "output"), p,
         _opt(w_index_ci, "w_index_ci"), _opt(w_index_co, "w_index_co"), weight.size(0), weight.size(1) * G)


def norm_dist_backward_input(grad_output, input, weight, output, grad_input, G, p, w_index_ci=None, w_index_co=None):
    B, CO, CI, HW = grad_output.size(0), output.size(1), input.size(1), input.size(2)
    _run("sd_norm_dist_backward_input", input, _chk(grad_output, "grad_output"), _chk(input, "input"),
         _chk(weight, "weight"), _chk(output, "output"), B, CO, CI, G, HW, _chk(grad_input, "grad_input"), p,
         _opt(w_index_ci, "w_index_ci"), _opt(w_index_co, "w_index_co"), weight.size(0), weight.size(1) * G)


def norm_dist_backward_input_weight(grad_output, input, weight, output, grad_input, grad_weight, G, p,
                                    w_index_ci=None, w_index_co=None):
    B, CO, CI, HW = grad_output.size(0), output.size(1), input.size(1), input.size(2)
    _run("sd_norm_dist_backward_input_weight", input, _chk(grad_output, "grad_output"), _chk(input, "input"),
         _chk(weight, "weight"), _chk(output, "output"), B, CO, CI, G, HW, _chk(grad_input, "grad_input"),
         _chk(grad_weight, "grad_weight"), p, _opt(w_index_ci, "w_index_ci"), _opt(w_index_co, "w_index_co"),
         weight.size(0), weight.size(1) * G)


def inf_dist_forward(input, weight, output, pos, G, w_index_ci=None, w_index_co=None):
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _run("sd_inf_dist_forward", input, _chk(input, "input"), _chk(weight, "weight"), B, CO, CI, G, HW,
         _chk(output, "output"), _chk(pos, "pos", torch.int32), _opt(w_index_ci, "w_index_ci"),
         _opt(w_index_co, "w_index_co"), weight.size(0), weight.size(1) * G)


def inf_dist_forward_nograd(input, weight, output, G):
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _run("sd_inf_dist_forward_nograd", input, _chk(input, "input"), _chk(weight, "weight"), B, CO, CI, G, HW,
         _chk(output, "output"))


def inf_dist_backward_input(grad_output, pos, grad_input, G):
    B, CO, CI, HW = grad_output.size(0), grad_output.size(1), grad_input.size(1), grad_input.size(2)
    _run("sd_inf_dist_backward_input", grad_output, _chk(grad_output, "grad_output"), _chk(pos, "pos", torch.int32),
         B, CO, CI, G, HW, _chk(grad_input, "grad_input"))


def inf_dist_backward_input_weight(grad_output, pos, grad_input, grad_weight, G, w_index_ci=None, w_index_co=None):
    B, CO, CI, HW = grad_output.size(0), grad_output.size(1), grad_input.size(1), grad_output.size(2)
    _run("sd_inf_dist_backward_input_weight", grad_output, _chk(grad_output, "grad_output"),
         _chk(pos, "pos", torch.int32), B, CO, CI, G, HW, _chk(grad_input, "grad_input"),
         _chk(grad_weight, "grad_weight"), _opt(w_index_ci, "w_index_ci"), _opt(w_index_co, "w_index_co"),
         grad_weight.size(0), grad_weight.size(1) * G)


def bound_inf_dist_forward_nograd(inputL, inputU, weight, outputL, outputU, G):
    B, CO, CI, HW = inputL.size(0), outputL.size(1), inputL.size(1), inputL.size(2)
    _run("sd_bound_inf_dist_forward_nograd", inputL, _chk(inputL, "inputL"), _chk(inputU, "inputU"),
         _chk(weight, "weight"), B, CO, CI, G, HW, _chk(outputL, "outputL"), _chk(outputU, "outputU"))


def bound_inf_dist_forward(inputL, inputU, weight, outputL, outputU, posL, posU, G):
    B, CO, CI, HW = inputL.size(0), outputL.size(1), inputL.size(1), inputL.size(2)
    _run("sd_bound_inf_dist_forward", inputL, _chk(inputL, "inputL"), _chk(inputU, "inputU"), _chk(weight, "weight"),
         B, CO, CI, G, HW, _chk(outputL, "outputL"), _chk(outputU, "outputU"),
         _chk(posL, "posL", torch.int32), _chk(posU, "posU", torch.int32))


def bound_inf_dist_backward_input(grad_outputL, grad_outputU, posL, posU, grad_inputL, grad_inputU, G):
    B, CO = grad_outputL.size(0), grad_outputL.size(1)
    CI, HW = grad_inputL.size(1), grad_inputL.size(2)
    _run("sd_bound_inf_dist_backward_input", grad_outputL, _chk(grad_outputL, "grad_outputL"),
         _chk(grad_outputU, "grad_outputU"), _chk(posL, "posL", torch.int32), _chk(posU, "posU", torch.int32),
         B, CO, CI, G, HW, _chk(grad_inputL, "grad_inputL"), _chk(grad_inputU, "grad_inputU"))


def bound_inf_dist_backward_input_weight(grad_outputL, grad_outputU, posL, posU, grad_inputL, grad_inputU,
                                         grad_weight, G):
    B, CO = grad_outputL.size(0), grad_outputL.size(1)
    CI, HW = grad_weight.size(1) * G, grad_outputL.size(2)
    _run("sd_bound_inf_dist_backward_input_weight", grad_outputL, _chk(grad_outputL, "grad_outputL"),
         _chk(grad_outputU, "grad_outputU"), _chk(posL, "posL", torch.int32), _chk(posU, "posU", torch.int32),
         B, CO, CI, G, HW, _chk(grad_inputL, "grad_inputL"), _chk(grad_inputU, "grad_inputU"),
         _chk(grad_weight, "grad_weight"))


def sort_neuron_forward(input, weight, output, pos, G, q, K):
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _run("sd_sort_neuron_forward", input, _chk(input, "input"), _chk(weight, "weight"), B, CO, CI, G, HW,
         _chk(output, "output"), _chk(pos, "pos", torch.int32), q, K)


def bound_sort_neuron_forward(inputL, inputU, weight, outputL, outputU, G, q, K):
    B, CO, CI, HW = inputL.size(0), outputL.size(1), inputL.size(1), inputL.size(2)
    _run("sd_bound_sort_neuron_forward", inputL, _chk(inputL, "inputL"), _chk(inputU, "inputU"),
         _chk(weight, "weight"), B, CO, CI, G, HW, _chk(outputL, "outputL"), _chk(outputU, "outputU"), q, K)


def sort_neuron_forward_nograd(input, weight, output, G, q, K):
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _run("sd_sort_neuron_forward_nograd", input, _chk(input, "input"), _chk(weight, "weight"), B, CO, CI, G, HW,
         _chk(output, "output"), q, K)


def sort_neuron_backward_input(grad_output, pos, grad_input, G, q, K):
    B, CO, CI, HW = grad_output.size(0), grad_output.size(1), grad_input.size(1), grad_input.size(2)
    _run("sd_sort_neuron_backward_input", grad_output, _chk(grad_output, "grad_output"),
         _chk(pos, "pos", torch.int32), B, CO, CI, G, HW, _chk(grad_input, "grad_input"), q, K)


def sort_neuron_backward_input_weight(grad_output, pos, grad_input, grad_weight, G, q, K):
    B, CO, CI, HW = grad_output.size(0), grad_output.size(1), grad_input.size(1), grad_output.size(2)
    _run("sd_sort_neuron_backward_input_weight", grad_output, _chk(grad_output, "grad_output"),
         _chk(pos, "pos", torch.int32), B, CO, CI, G, HW, _chk(grad_input, "grad_input"),
         _chk(grad_weight, "grad_weight"), q, K)


def masked_inf_dist_forward(input, weight, output, pos, G, q, seed, mode=MASK_TERM):
    """Not in the reference extension: max over a Bernoulli(q)-kept subset of |input - weight|
    with the keep decisions drawn from the library's counter RNG; pos may be None."""
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _run("sd_masked_inf_dist_forward", input, _chk(input, "input"), _chk(weight, "weight"), B, CO, CI, G, HW,
         _chk(output, "output"), None if pos is None else _chk(pos, "pos", torch.int32), q, seed & 0xFFFFFFFF, mode)


def mean_shift_forward(input, mean, running_mean, momentum, output):
    """Not in the reference extension (done there with torch ops): mean over batch and positions,
    optional in-place running-mean update, output = input - mean."""
    B, C, HW = input.size(0), input.size(1), input.size(2)
    _run("sd_mean_shift_forward", input, _chk(input, "input"), B, C, HW, _chk(mean, "mean"),
         None if running_mean is None else _chk(running_mean, "running_mean"), momentum, _chk(output, "output"))


def mean_shift_index_forward(input, index, channels_per_group, mean, running_mean, momentum, output):
    """Not in the reference extension (done there with torch ops): training-mode mean shift of a
    (B, G * cnt, HW) tensor that holds, per 32-sample sub-batch, the channels index[s, g, :] of
    `channels_per_group` channels per group."""
    B, HW = input.size(0), input.size(2)
    G, cnt = index.size(-2), index.size(-1)
    _run("sd_mean_shift_index_forward", input, _chk(input, "input"), _chk(index, "index", torch.int32), B, G, cnt,
         channels_per_group, HW, _chk(mean, "mean"),
         None if running_mean is None else _chk(running_mean, "running_mean"), momentum, _chk(output, "output"))


def channel_shift(input, shift, sign, output):
    """output = input + sign * shift[c] (evaluation-mode mean shift, bias add)."""
    B, C, HW = input.size(0), input.size(1), input.size(2)
    _run("sd_channel_shift", input, _chk(input, "input"), _chk(shift, "shift"), B, C, HW, sign, _chk(output, "output"))


def rng_word(seed, stream, row, col):
    """One 32-bit word of the library's counter RNG (host arithmetic; the kernels use the same function)."""
    return int(_lib.load().sd_rng_word(seed & 0xFFFFFFFF, stream, row & 0xFFFFFFFF, col & 0xFFFFFFFF))


def mask_count(seed, channels, q):
    """Number of kept channels for keep probability q (host arithmetic only, no GPU work)."""
    return int(_lib.load().sd_mask_count(seed & 0xFFFFFFFF, channels, q))


def sample_index_lists(seed, sub_batches, groups, channels, count, device):
    """(sub_batches, groups, count) int32 tensor of ascending kept-channel indices, drawn on the
    device from the counter RNG (the reference's sample_mask without its host synchronisation)."""
    out = torch.empty(sub_batches, groups, count, device=device, dtype=torch.int32)
    if count > 0:
        with torch.cuda.device(out.device):
            _lib.call("sd_sample_index_lists", seed & 0xFFFFFFFF, sub_batches, groups, channels, count,
                      out.data_ptr(), torch.cuda.current_stream(out.device).cuda_stream)
    return out

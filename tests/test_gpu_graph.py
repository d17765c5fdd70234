"""HIP graph capture of the library's entry points: a sequence of forward and backward calls is captured once
(after an eager warm-up, so that the library workspace already has its size and nothing allocates under capture)
and replayed several times on new input contents, with eager work between the replays; every replay must
reproduce the eager results (bit for bit for the l-inf values and positions, to the gradient tolerance for the
atomically accumulated sums).  The library zero-fills with a kernel, never a memset node."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _close(a, b, what):
    a, b = a.cpu().numpy(), b.cpu().numpy()
    np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-5 * max(float(np.abs(b).max()), 1e-30), err_msg=what)


def test_graph_replays_match_eager():
    from sortnet_amd import ext
    dev = _dev()
    B, CI, CO, K = 96, 1024, 320, 6
    g = torch.Generator().manual_seed(5)
    S = (B + 31) // 32
    cn, cm = ext.mask_count(11, CI, 0.6), ext.mask_count(12, CO, 0.6)
    ci = ext.sample_index_lists(11, S, 1, CI, cn, dev)
    co = ext.sample_index_lists(12, S, 1, CO, cm, dev)

    x = torch.empty(B, CI, 1, device=dev); w = torch.empty(CO, CI, device=dev); gy = torch.empty(B, CO, 1, device=dev)
    xc = torch.empty(B, cn, 1, device=dev); gyc = torch.empty(B, cm, 1, device=dev)

    def outputs():
        return dict(
            y=torch.empty(B, CO, 1, device=dev), pos=torch.empty(B, CO, 1, device=dev, dtype=torch.int32),
            gx=torch.empty_like(x), gw=torch.empty_like(w),
            yl=torch.empty(B, CO, 1, device=dev), yu=torch.empty(B, CO, 1, device=dev),
            ys=torch.empty(B, CO, 1, device=dev),
            yp=torch.empty(B, CO, 1, device=dev), gxp=torch.empty_like(x), gwp=torch.empty_like(w),
            yc=torch.empty(B, cm, 1, device=dev), posc=torch.empty(B, cm, 1, device=dev, dtype=torch.int32),
            gxc=torch.empty_like(xc), gwc=torch.empty_like(w),
            ypc=torch.empty(B, cm, 1, device=dev), gxpc=torch.empty_like(xc), gwpc=torch.empty_like(w))

    def run(o):
        ext.inf_dist_forward(x, w, o["y"], o["pos"], 1)
        ext.inf_dist_backward_input_weight(gy, o["pos"], o["gx"], o["gw"], 1)
        ext.bound_inf_dist_forward_nograd(x - 0.05, x + 0.05, w, o["yl"], o["yu"], 1)
        ext.sort_neuron_forward_nograd(x, w, o["ys"], 1, 0.4, K)
        ext.norm_dist_forward(x, w, o["yp"], 1, 8.0)
        ext.norm_dist_backward_input_weight(gy, x, w, o["yp"], o["gxp"], o["gwp"], 1, 8.0)
        ext.inf_dist_forward(xc, w, o["yc"], o["posc"], 1, ci, co)
        ext.inf_dist_backward_input_weight(gyc, o["posc"], o["gxc"], o["gwc"], 1, ci, co)
        ext.norm_dist_forward(xc, w, o["ypc"], 1, 12.5, ci, co)
        ext.norm_dist_backward_input_weight(gyc, xc, w, o["ypc"], o["gxpc"], o["gwpc"], 1, 12.5, ci, co)

    def new_inputs(scale):
        x.copy_(torch.rand(B, CI, 1, generator=g) * scale); w.copy_(torch.randn(CO, CI, generator=g) * 0.2)
        gy.copy_(torch.randn(B, CO, 1, generator=g)); xc.copy_(torch.rand(B, cn, 1, generator=g) * scale)
        gyc.copy_(torch.randn(B, cm, 1, generator=g))

    new_inputs(1.0)
    eager = outputs()
    run(eager)                      # warm-up: workspace growth and one-time queries happen here
    torch.cuda.synchronize()

    captured = outputs()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(captured)

    exact = ("y", "pos", "yl", "yu", "yc", "posc")
    for replay, scale in enumerate((1.0, 0.5, 2.0, 1.0)):
        new_inputs(scale)
        run(eager)                  # the program's own eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name in eager:
            if name in exact:
                assert torch.equal(eager[name], captured[name]), "%s, replay %d" % (name, replay)
            else:
                _close(captured[name], eager[name], "%s, replay %d" % (name, replay))

"""sd_time_forward_kernels / sd_last_forward_kernel_ms: the events the library records around a forward tile
kernel's own launch (bench.py takes its roofline figures from them)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_forward_kernel_timer_reports_the_tile_kernel():
    from sortnet_amd import _lib, ext
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    B, CI, CO = 256, 1024, 512
    x = torch.rand(B, CI, 1, generator=g).to(dev)
    w = torch.randn(CO, CI, generator=g).to(dev)
    y = torch.empty(B, CO, 1, device=dev)
    pos = torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
    _lib.time_forward_kernels(False)
    ext.inf_dist_forward_nograd(x, w, y, 1)
    assert _lib.last_forward_kernel_ms() is None
    _lib.time_forward_kernels(True)
    try:
        assert _lib.last_forward_kernel_ms() is None          # nothing timed yet
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for call in (lambda: ext.inf_dist_forward_nograd(x, w, y, 1),
                     lambda: ext.inf_dist_forward(x, w, y, pos, 1),
                     lambda: ext.masked_inf_dist_forward(x, w, y, pos, 1, 0.3, 5, ext.MASK_FACTORED),
                     lambda: ext.bound_inf_dist_forward_nograd(x, x + 0.01, w, y, torch.empty_like(y), 1)):
            e0.record()
            call()
            e1.record()
            ms = _lib.last_forward_kernel_ms()
            torch.cuda.synchronize()
            assert ms is not None and 0.0 < ms <= e0.elapsed_time(e1) + 1e-3, ms
    finally:
        _lib.time_forward_kernels(False)
    assert _lib.last_forward_kernel_ms() is None

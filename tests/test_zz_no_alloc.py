"""The entry point that allocates nothing (sd_inf_dist_forward_noalloc) against sd_inf_dist_forward, through
the C ABI: values and positions bit for bit, on two calls in a row that share the built-in scratch array, the
second one smaller than the first (stale merge keys of the first call must not leak into it); and the property the
entry point exists for: a call leaves the device's free memory unchanged, on a stream the library has never seen
(no workspace of its own), and it can be recorded into a graph and replayed."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _call(name, x, w, y, pos, ci=None, co=None, G=1):
    from sortnet_amd import _lib
    B, CI, HW = x.shape
    CO = y.size(1)
    with torch.cuda.device(x.device):
        _lib.call(name, x.data_ptr(), w.data_ptr(), B, CO, CI, G, HW, y.data_ptr(), pos.data_ptr(),
                  None if ci is None else ci.data_ptr(), None if co is None else co.data_ptr(),
                  w.size(0), w.size(1) * G, torch.cuda.current_stream(x.device).cuda_stream)


def _pair(B, CI, CO, seed, dev, grid=None):
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(B, CI, 1, generator=g)
    w = torch.randn(CO, CI, generator=g) * 0.3
    if grid:   # coarse values: many exact ties, so the lowest-index rule is exercised through the merge
        x, w = (x * grid).round() / grid, (w * grid).round() / grid
    return x.to(dev), w.to(dev)


def _both(x, w, **kw):
    out = []
    for name in ("sd_inf_dist_forward", "sd_inf_dist_forward_noalloc"):
        CO = kw["co"].size(-1) if kw.get("co") is not None else w.size(0)
        y = torch.full((x.size(0), CO, 1), -1.0, device=x.device)
        pos = torch.full((x.size(0), CO, 1), -7, device=x.device, dtype=torch.int32)
        _call(name, x, w, y, pos, **kw)
        out.append((y, pos))
    torch.cuda.synchronize()
    return out


def test_noalloc_matches_inf_dist_forward_twice():
    dev = _dev()
    # split reduction on both calls (few output tiles, long rows); the second is smaller in every dimension
    for B, CI, CO, seed, grid in [(128, 3072, 1024, 11, None), (48, 1024, 320, 12, 8)]:
        x, w = _pair(B, CI, CO, seed, dev, grid)
        (y0, p0), (y1, p1) = _both(x, w)
        assert torch.equal(y0, y1), (B, CI, CO)
        assert torch.equal(p0, p1), (B, CI, CO)
        assert float(y0.min()) > 0


def test_noalloc_index_lists_and_limit():
    import numpy as np
    from sortnet_amd import _lib
    dev = _dev()
    B, CI, CO = 64, 512, 256
    x, w = _pair(B, 200, CO, 13, dev)          # compacted input: 200 kept of 512 columns
    wfull = torch.randn(CO, CI, generator=torch.Generator().manual_seed(14)).to(dev)
    rng = np.random.default_rng(5)
    ci = torch.tensor(np.stack([[np.sort(rng.choice(CI, 200, replace=False))] for _ in range(2)]).astype(np.int32)).to(dev)
    co = torch.tensor(np.stack([[np.sort(rng.choice(CO, 96, replace=False))] for _ in range(2)]).astype(np.int32)).to(dev)
    (y0, p0), (y1, p1) = _both(x, wfull, ci=ci, co=co)
    assert torch.equal(y0, y1) and torch.equal(p0, p1)
    # beyond the built-in scratch: rejected before anything is launched (no buffer is touched)
    with pytest.raises(RuntimeError, match="exceed the maximum"):
        _lib.call("sd_inf_dist_forward_noalloc", x.data_ptr(), w.data_ptr(), 4096, 2048, 200, 1, 1,
                  x.data_ptr(), x.data_ptr(), None, None, 0, 0, None)


def test_noalloc_allocates_nothing_and_runs_under_capture():
    dev = _dev()
    x, w = _pair(128, 3072, 1024, 21, dev)           # split reduction: the merge scratch is in use
    (y0, p0), _ = _both(x, w)                         # reference result; also warms up code objects and the scratch address
    y = torch.full_like(y0, -1.0)
    pos = torch.full_like(p0, -7)
    fresh = torch.cuda.Stream(device=dev)             # the library holds no workspace for this stream
    with torch.cuda.stream(fresh):                    # (whatever the runtime sets up at a stream's first launch: now)
        torch.zeros(8, device=dev).add_(1)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info(dev)
    with torch.cuda.stream(fresh):
        _call("sd_inf_dist_forward_noalloc", x, w, y, pos)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info(dev)
    assert free1 == free0, "the call changed the device's free memory by %d bytes" % (free0 - free1)
    assert torch.equal(y, y0) and torch.equal(pos, p0)
    # recorded into a graph (where hipMalloc is not allowed) and replayed, with eager work between the replays
    y.fill_(-1.0)
    pos.fill_(-7)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _call("sd_inf_dist_forward_noalloc", x, w, y, pos)
    for k in range(3):
        y.fill_(-1.0)
        pos.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, y0) and torch.equal(pos, p0), "replay %d" % k
        (e0, q0), _ = _both(x, w)                     # eager calls that share the scratch, between replays
        assert torch.equal(e0, y0) and torch.equal(q0, p0)

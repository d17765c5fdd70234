"""HIP graph capture of the library's entry points, and calls that overlap on two streams.

A sequence of forward and backward calls is captured once (after an eager warm-up on the capture stream, so
that this stream's library workspace already has its size and nothing allocates under capture) and replayed
several times on new input contents, with eager work between the replays; every replay must reproduce the eager
results (bit for bit for the l-inf values and positions, to the gradient tolerance for the atomically
accumulated sums).  The library zero-fills with a kernel, never a memset node.  The workspace is kept per
(device, stream), so calls queued on two streams may overlap: the second test checks that."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _built_in_limits_afterwards():
    """A test that sets a candidate-table limit by hand leaves the built-in ones behind, pass or fail."""
    yield
    from sortnet_amd import _lib
    _lib.set_bound_candidate_density(-1.0)
    _lib.set_linf_candidate_density(-1.0)
    _lib.set_sort_candidate_density(-1.0)


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
    captured = outputs()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(captured)               # warm-up on the capture stream: its workspace grows here, not under capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
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


def test_calls_on_two_streams_overlap_safely(oracle):
    """Two streams run workspace-using calls of different sizes at the same time (split-reduction merges of the
    position kernels, the two-level sort neuron, l-p partial sums); each result must equal the one the same call
    gives alone."""
    from sortnet_amd import ext
    dev = _dev()
    g = torch.Generator().manual_seed(9)

    def make(B, CI, CO):
        x = torch.rand(B, CI, 1, generator=g).to(dev); w = (torch.randn(CO, CI, generator=g) * 0.2).to(dev)
        return x, w, dict(y=torch.empty(B, CO, 1, device=dev), pos=torch.empty(B, CO, 1, device=dev, dtype=torch.int32),
                          ys=torch.empty(B, CO, 1, device=dev), yp=torch.empty(B, CO, 1, device=dev))

    def run(x, w, o):
        ext.inf_dist_forward(x, w, o["y"], o["pos"], 1)
        ext.sort_neuron_forward_nograd(x, w, o["ys"], 1, 0.4, 5)
        ext.norm_dist_forward(x, w, o["yp"], 1, 24.0)

    xa, wa, oa = make(64, 4096, 96)       # few output tiles: split reductions, partial sums in the workspace
    xb, wb, ob = make(40, 2048, 200)
    _, _, ra = make(64, 4096, 96); _, _, rb = make(40, 2048, 200)
    run(xa, wa, ra); run(xb, wb, rb)
    torch.cuda.synchronize()
    ry, rpos = oracle.inf_dist_forward(xa.cpu().numpy(), wa.cpu().numpy())
    assert np.array_equal(ra["y"].cpu().numpy(), ry) and np.array_equal(ra["pos"].cpu().numpy(), rpos)

    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    for _ in range(20):
        with torch.cuda.stream(sa):
            run(xa, wa, oa)
        with torch.cuda.stream(sb):
            run(xb, wb, ob)
    torch.cuda.synchronize()
    for got, want in ((oa, ra), (ob, rb)):
        assert torch.equal(got["y"], want["y"]) and torch.equal(got["pos"], want["pos"])
        _close(got["ys"], want["ys"], "sort neuron"); _close(got["yp"], want["yp"], "l-p")


def test_graph_replays_of_the_lds_direct_kernels():
    """The same protocol at a shape that takes the LDS-direct kernels (exact 64 x 128 tiles, split reduction range):
    l-inf with and without positions, the factored-mask neuron, the interval forward and the l-p forward, captured once
    and replayed on new contents; all of them bit for bit against eager calls except the l-p sums (rel 1e-5)."""
    from sortnet_amd import ext, _lib
    dev = _dev()
    B, CI, CO = 256, 2048, 2048
    g = torch.Generator().manual_seed(15)
    x = torch.empty(B, CI, 1, device=dev); w = torch.empty(CO, CI, device=dev)

    def outputs():
        f = lambda: torch.empty(B, CO, 1, device=dev)
        i = lambda: torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
        return dict(y=f(), pos=i(), yn=f(), ym=f(), pm=i(), yl=f(), yu=f(), yp=f())

    def run(o):
        names = []
        ext.inf_dist_forward(x, w, o["y"], o["pos"], 1); names.append(_lib.last_forward_kernel())
        ext.inf_dist_forward_nograd(x, w, o["yn"], 1); names.append(_lib.last_forward_kernel())
        ext.masked_inf_dist_forward(x, w, o["ym"], o["pm"], 1, 0.3, 21, ext.MASK_FACTORED); names.append(_lib.last_forward_kernel())
        ext.bound_inf_dist_forward_nograd(x - 0.05, x + 0.05, w, o["yl"], o["yu"], 1); names.append(_lib.last_forward_kernel())
        ext.norm_dist_forward(x, w, o["yp"], 1, 8.0); names.append(_lib.last_forward_kernel())
        return names

    def new_inputs(scale):
        x.copy_(torch.rand(B, CI, 1, generator=g) * scale); w.copy_(torch.randn(CO, CI, generator=g) * 0.2)

    new_inputs(1.0)
    eager, captured = outputs(), outputs()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        names = run(captured)       # warm-up on the capture stream sizes its workspace
    assert all(n == "fwd_kernel_direct<4,8>" for n in names), names
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(captured)
    for replay, scale in enumerate((1.0, 0.5, 2.0)):
        new_inputs(scale)
        run(eager)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name in eager:
            if name == "yp":
                _close(captured[name], eager[name], "%s, replay %d" % (name, replay))
            else:
                assert torch.equal(eager[name], captured[name]), "%s, replay %d" % (name, replay)


def test_graph_replays_of_the_candidate_table_kernels(oracle):
    """Dense l-p calls at general p (and the interval forward, the sort neuron and its interval bounds) queue a
    candidate-table kernel and an every-term kernel for the same result and a count taken on the device picks one, so ONE captured graph serves both kinds of data: replays on weights far
    smaller than the inputs (the table kernel runs) and on weights as large as the inputs (the every-term kernels
    run) must both reproduce eager calls, and the oracle."""
    from sortnet_amd import ext, _lib
    dev = _dev()
    B, CI, CO, p = 160, 1024, 300, 64.0
    g = torch.Generator().manual_seed(25)
    # the interval forward's built-in limits leave layers of this size to the every-term kernel: a limit set by hand
    # applies at any size, and the count on the device still decides between the two kernels
    _lib.set_bound_candidate_density(0.25)
    x = torch.empty(B, CI, 1, device=dev); w = torch.empty(CO, CI, device=dev); gy = torch.empty(B, CO, 1, device=dev)

    def outputs():
        return dict(y=torch.empty(B, CO, 1, device=dev), gx=torch.empty_like(x), gw=torch.empty_like(w),
                    gx2=torch.empty_like(x), yl=torch.empty(B, CO, 1, device=dev), yu=torch.empty(B, CO, 1, device=dev),
                    ys=torch.empty(B, CO, 1, device=dev), ysl=torch.empty(B, CO, 1, device=dev),
                    ysu=torch.empty(B, CO, 1, device=dev), zl=torch.empty(B, CO, 1, device=dev),
                    zu=torch.empty(B, CO, 1, device=dev), pl=torch.empty(B, CO, 1, device=dev, dtype=torch.int32),
                    pu=torch.empty(B, CO, 1, device=dev, dtype=torch.int32))

    def run(o):
        # the interval forward makes the same kind of choice (rows of the batch alike or not)
        ext.bound_inf_dist_forward_nograd(x - 0.03, x + 0.03, w, o["yl"], o["yu"], 1)
        ext.bound_inf_dist_forward(x - 0.03, x + 0.03, w, o["zl"], o["zu"], o["pl"], o["pu"], 1)
        # so do the sort neuron and its interval bounds
        ext.sort_neuron_forward_nograd(x, w, o["ys"], 1, 0.5, 6)
        ext.bound_sort_neuron_forward(x - 0.03, x + 0.03, w, o["ysl"], o["ysu"], 1, 0.5, 6)
        ext.norm_dist_forward(x, w, o["y"], 1, p)
        ext.norm_dist_backward_input_weight(gy, x, w, o["y"], o["gx"], o["gw"], 1, p)
        ext.norm_dist_backward_input(gy, x, w, o["y"], o["gx2"], 1, p)

    def new_inputs(wscale):
        # small weights come with batch rows that are nearly alike, large weights with unrelated rows
        base = torch.randn(1, CI, 1, generator=g) if wscale < 0.1 else 0.0
        x.copy_(base + torch.randn(B, CI, 1, generator=g) * (0.01 if wscale < 0.1 else 1.0))
        w.copy_(torch.randn(CO, CI, generator=g) * wscale)
        gy.copy_(torch.randn(B, CO, 1, generator=g))

    new_inputs(0.02)
    eager, captured = outputs(), outputs()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(captured)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(captured)
    for replay, wscale in enumerate((0.02, 1.0, 0.02, 1.5)):
        new_inputs(wscale)
        run(eager)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name in eager:
            if name in ("yl", "yu", "ys", "ysl", "ysu", "zl", "zu", "pl", "pu"):
                assert torch.equal(captured[name], eager[name]), "%s, replay %d" % (name, replay)
                continue
            a, b = captured[name].cpu().numpy(), eager[name].cpu().numpy()
            np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-4 * float(np.abs(b).max()), err_msg="%s, replay %d" % (name, replay))
        rl, ru = oracle.bound_inf_dist_forward((x - 0.03).cpu().numpy(), (x + 0.03).cpu().numpy(), w.cpu().numpy(), 1, need_pos=False)
        assert np.array_equal(captured["yl"].cpu().numpy(), rl) and np.array_equal(captured["yu"].cpu().numpy(), ru), replay
        _, _, rpl, rpu = oracle.bound_inf_dist_forward((x - 0.03).cpu().numpy(), (x + 0.03).cpu().numpy(), w.cpu().numpy(), 1, need_pos=True)
        assert np.array_equal(captured["zl"].cpu().numpy(), rl) and np.array_equal(captured["zu"].cpu().numpy(), ru), replay
        assert np.array_equal(captured["pl"].cpu().numpy(), rpl) and np.array_equal(captured["pu"].cpu().numpy(), rpu), replay
        rs = oracle.sort_neuron_forward(x.cpu().numpy(), w.cpu().numpy(), 0.5, 6, need_pos=False)
        np.testing.assert_allclose(captured["ys"].cpu().numpy(), rs, rtol=1e-5, err_msg="replay %d" % replay)
        rsl, rsu = oracle.bound_sort_neuron_forward((x - 0.03).cpu().numpy(), (x + 0.03).cpu().numpy(), w.cpu().numpy(), 0.5, 6)
        np.testing.assert_allclose(captured["ysl"].cpu().numpy(), rsl, rtol=1e-5, err_msg="replay %d" % replay)
        np.testing.assert_allclose(captured["ysu"].cpu().numpy(), rsu, rtol=1e-5, err_msg="replay %d" % replay)
        ry = oracle.norm_dist_forward(x.cpu().numpy(), w.cpu().numpy(), p, 1)
        np.testing.assert_allclose(captured["y"].cpu().numpy(), ry, rtol=1e-5, err_msg="replay %d" % replay)
        rgx, rgw = oracle.norm_dist_backward(gy.cpu().numpy(), x.cpu().numpy(), w.cpu().numpy(), ry, p, 1)
        # the kernels differentiated their own y, which agrees with the oracle's to rel 1e-5: (d/y)^(p-1) moves by p times that
        for got, ref in ((captured["gx"], rgx), (captured["gw"], rgw), (captured["gx2"], rgx)):
            np.testing.assert_allclose(got.cpu().numpy(), ref, rtol=2e-3, atol=2e-3 * float(np.abs(ref).max()))


def test_graph_replays_of_both_table_orientations():
    """The l-inf forward, the masked neuron, the sort neuron with positions and the interval forward with positions
    queue the kernels of the tables per weight row, of the tables per batch row and the every-term kernels for one
    result, and counts taken on the device pick one.  ONE captured graph must therefore serve batch rows that are alike
    against weights of unit scale (tables per weight row), images against small weights (tables per batch row) and
    unrelated rows (every term): every replay reproduces the eager calls and the calls with every table switched off,
    bit for bit, values and positions."""
    from sortnet_amd import ext, _lib
    dev = _dev()
    B, CI, CO, K = 160, 1024, 300, 6
    g = torch.Generator().manual_seed(31)
    x = torch.empty(B, CI, 1, device=dev); w = torch.empty(CO, CI, device=dev)

    def limits(d):
        _lib.set_bound_candidate_density(d); _lib.set_linf_candidate_density(d); _lib.set_sort_candidate_density(d)

    def outputs():
        f = lambda: torch.empty(B, CO, 1, device=dev)
        i = lambda: torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
        return dict(y=f(), pos=i(), ym=f(), pm=i(), ys=f(), pk=torch.empty(K, B, CO, 1, device=dev, dtype=torch.int32),
                    zl=f(), zu=f(), pl=i(), pu=i(), ysl=f(), ysu=f())

    def run(o):
        ext.inf_dist_forward(x, w, o["y"], o["pos"], 1)
        ext.masked_inf_dist_forward(x, w, o["ym"], o["pm"], 1, 0.3, 9, ext.MASK_FACTORED)
        ext.sort_neuron_forward(x, w, o["ys"], o["pk"], 1, 0.5, K)
        ext.bound_inf_dist_forward(x - 0.03, x + 0.03, w, o["zl"], o["zu"], o["pl"], o["pu"], 1)
        ext.bound_sort_neuron_forward(x - 0.03, x + 0.03, w, o["ysl"], o["ysu"], 1, 0.5, K)

    def new_inputs(kind):
        if kind == "alike":
            x.copy_(torch.randn(1, CI, 1, generator=g) * 0.3 + torch.randn(B, CI, 1, generator=g) * 0.02)
            w.copy_(torch.randn(CO, CI, generator=g))
        elif kind == "images":
            x.copy_(torch.rand(B, CI, 1, generator=g))
            w.copy_(torch.randn(CO, CI, generator=g) * CI ** -0.5)
        else:
            x.copy_(torch.randn(B, CI, 1, generator=g))
            w.copy_(torch.randn(CO, CI, generator=g))

    limits(0.5)   # a limit set by hand applies at any size; the counts on the device still decide
    new_inputs("images")
    eager, captured, plain = outputs(), outputs(), outputs()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(captured)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(captured)
    served = {}
    for replay, kind in enumerate(("images", "alike", "random", "images", "alike")):
        new_inputs(kind)
        run(eager)
        served[kind] = _lib.last_forward_term_share()    # of the last call, the interval sort neuron
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        limits(0.0)
        run(plain)
        torch.cuda.synchronize()
        limits(0.5)
        for name in eager:
            assert torch.equal(captured[name], eager[name]), "%s, replay %d (%s): graph against eager" % (name, replay, kind)
            assert torch.equal(captured[name], plain[name]), "%s, replay %d (%s): tables against every term" % (name, replay, kind)
    assert served["images"] < 1.0 and served["alike"] < 1.0 and served["random"] == 1.0, served


def test_two_host_threads_on_one_stream_leave_results_unchanged():
    """Two host threads call the same layers at the same time on torch's default stream (which all threads share
    unless they switch): every entry point that uses the stream's workspace - split-reduction merge buffers, keep bits,
    candidate tables - must give each thread the results it gets alone, call after call."""
    import threading
    from sortnet_amd import ext, _lib
    dev = _dev()
    B, CI, CO = 128, 3072, 384
    _lib.set_bound_candidate_density(0.25)            # tables at this size, the count on the device still decides
    w = (torch.randn(CO, CI, generator=torch.Generator().manual_seed(40)) * CI ** -0.5).to(dev)

    def inputs(seed):
        g = torch.Generator().manual_seed(seed)
        base = torch.randn(1, CI, 1, generator=g) * 0.1
        return (base + torch.randn(B, CI, 1, generator=g) * (0.01 if seed % 2 else 0.2)).to(dev)

    def run(x, n):
        outs = []
        for _ in range(n):
            y = torch.empty(B, CO, 1, device=dev); pos = torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
            ym = torch.empty_like(y); pm = torch.empty_like(pos)
            yl, yu = torch.empty_like(y), torch.empty_like(y)
            zl, zu, pl, pu = torch.empty_like(y), torch.empty_like(y), torch.empty_like(pos), torch.empty_like(pos)
            ys = torch.empty_like(y)
            ext.inf_dist_forward(x, w, y, pos, 1)
            ext.masked_inf_dist_forward(x, w, ym, pm, 1, 0.3, 5, ext.MASK_FACTORED)
            ext.bound_inf_dist_forward_nograd(x - 0.02, x + 0.02, w, yl, yu, 1)
            ext.bound_inf_dist_forward(x - 0.02, x + 0.02, w, zl, zu, pl, pu, 1)
            ext.sort_neuron_forward_nograd(x, w, ys, 1, 0.5, 6)
            outs.append((y, pos, ym, pm, yl, yu, zl, zu, pl, pu, ys))
        return outs

    xs = [inputs(1), inputs(2)]
    alone = [run(x, 1)[0] for x in xs]
    torch.cuda.synchronize()
    got, errors = [None, None], []

    def worker(i):
        try:
            torch.cuda.set_device(dev)
            got[i] = run(xs[i], 12)
        except Exception as e:      # noqa: BLE001 - reported by the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for i in range(2):
        for k, outs in enumerate(got[i]):
            for a, b in zip(outs, alone[i]):
                assert torch.equal(a, b), "thread %d, call %d" % (i, k)

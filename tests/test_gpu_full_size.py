"""GPU parity at the full benchmark shapes.

The scalar oracle cannot run 13.4 G terms inside a test, but every forward output row depends only
on its own input row, so the first ROWS samples of a full-size launch are compared with the oracle
run on those samples alone (same weights, same row numbers, hence the same counter-RNG masks).
Batch-summed results (grad_weight) are compared with an independent accumulation of the same
quantities on a slice of weight rows.  Bit-exact sets use array_equal, the others rel 1e-5.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL = 1e-5
ROWS = 12


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _close(got, ref, rtol=RTOL):
    got = got.cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got)
    ref = ref.cpu().numpy() if isinstance(ref, torch.Tensor) else np.asarray(ref)
    np.testing.assert_allclose(got, ref, rtol=rtol, atol=rtol * max(float(np.abs(ref).max()), 1e-30))


def _inputs(B, N, M, kind, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(B, N, generator=g) if kind == "rand" else torch.randn(B, N, generator=g)
    w = torch.randn(M, N, generator=g) * N ** -0.5
    gy = torch.randn(B, M, generator=g)
    return x.unsqueeze(-1).contiguous(), w.contiguous(), gy.unsqueeze(-1).contiguous()


def _scatter_reference(gy, pos, B, N, M, dev):
    """grad_x / grad_w of the scatter backward from torch index_put_ on the device."""
    idx = (pos & 0x7FFFFFFF).long().view(B, M)
    s = torch.where(pos.view(B, M) < 0, -gy.view(B, M), gy.view(B, M))
    gx = torch.zeros(B, N, device=dev).scatter_add_(1, idx, s)
    rows = torch.arange(M, device=dev).view(1, M).expand(B, M)
    gw = torch.zeros(M, N, device=dev).index_put_((rows.reshape(-1), idx.reshape(-1)), -s.reshape(-1), accumulate=True)
    return gx, gw


def test_masked_layer_512x5120x5120(oracle):
    """Masked order-statistic layer, B=512, N=M=5120, q=0.3: dense, per-term and factored masks with
    positions; interval bounds for [x-2/255, x+2/255] with positions; scatter backward of all of them."""
    from sortnet_amd import ext
    dev = _dev()
    B = 512
    N = M = 5120
    x, w, gy = _inputs(B, N, M, "rand")
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    xs, wn = x[:ROWS].numpy(), w.numpy()
    y = torch.empty(B, M, 1, device=dev)
    yn = torch.empty_like(y)
    pos = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)

    ext.inf_dist_forward(xd, wd, y, pos, 1)
    ext.inf_dist_forward_nograd(xd, wd, yn, 1)
    ry, rpos = oracle.inf_dist_forward(xs, wn)
    assert np.array_equal(y[:ROWS].cpu().numpy(), ry) and np.array_equal(pos[:ROWS].cpu().numpy(), rpos)
    assert torch.equal(y, yn)
    ext.inf_dist_backward_input_weight(gd, pos, gx, gw, 1)
    tgx, tgw = _scatter_reference(gd, pos, B, N, M, dev)
    _close(gx.view(B, N), tgx)
    _close(gw, tgw)
    rgx = oracle.inf_dist_backward(gy[:ROWS].numpy(), rpos, xs.shape, wn.shape, need_weight=False)
    _close(gx[:ROWS], rgx)

    for mode in (ext.MASK_TERM, ext.MASK_FACTORED):
        ext.masked_inf_dist_forward(xd, wd, y, pos, 1, 0.3, 7, mode)
        ext.masked_inf_dist_forward(xd, wd, yn, None, 1, 0.3, 7, mode)
        ry, rpos = oracle.masked_inf_dist_forward(xs, wn, 0.3, 7, mode)
        assert np.array_equal(y[:ROWS].cpu().numpy(), ry), mode
        assert np.array_equal(pos[:ROWS].cpu().numpy(), rpos), mode
        assert torch.equal(y, yn), mode

    eps = np.float32(2.0 / 255)
    xl, xu = (x - eps).contiguous(), (x + eps).contiguous()
    xld, xud = xl.to(dev), xu.to(dev)
    yl, yu = torch.empty_like(y), torch.empty_like(y)
    yl2, yu2 = torch.empty_like(y), torch.empty_like(y)
    pl, pu = torch.empty_like(pos), torch.empty_like(pos)
    ext.bound_inf_dist_forward(xld, xud, wd, yl, yu, pl, pu, 1)
    ext.bound_inf_dist_forward_nograd(xld, xud, wd, yl2, yu2, 1)
    ryl, ryu, rpl, rpu = oracle.bound_inf_dist_forward(xl[:ROWS].numpy(), xu[:ROWS].numpy(), wn)
    for got, ref in ((yl, ryl), (yu, ryu), (pl, rpl), (pu, rpu)):
        assert np.array_equal(got[:ROWS].cpu().numpy(), ref)
    assert torch.equal(yl, yl2) and torch.equal(yu, yu2)
    gl = torch.randn(B, M, 1, generator=torch.Generator().manual_seed(1)).to(dev)
    gxl, gxu = torch.empty_like(xd), torch.empty_like(xd)
    ext.bound_inf_dist_backward_input_weight(gl, gd, pl, pu, gxl, gxu, gw, 1)
    rgxl, rgxu = oracle.bound_inf_dist_backward(gl[:ROWS].cpu().numpy(), gy[:ROWS].numpy(), rpl, rpu, xs.shape,
                                                wn.shape, need_weight=False)
    _close(gxl[:ROWS], rgxl)
    _close(gxu[:ROWS], rgxu)
    # every unit of upstream gradient lands somewhere in grad_w with its sign flipped or kept
    assert float(gw.abs().sum()) <= float(gl.abs().sum() + gd.abs().sum()) * (1 + 1e-4)


def test_sort_neuron_512x5120x5120(oracle):
    """Evaluation form of the same layer (top-10 weighted order statistics) and its interval version."""
    from sortnet_amd import ext
    dev = _dev()
    B = 512
    N = M = 5120
    K, q = 10, 0.3
    x, w, gy = _inputs(B, N, M, "rand")
    xd, wd = x.to(dev), w.to(dev)
    xs, wn = x[:ROWS].numpy(), w.numpy()
    y = torch.empty(B, M, 1, device=dev)
    yn = torch.empty_like(y)
    pos = torch.empty(K, B, M, 1, device=dev, dtype=torch.int32)
    ext.sort_neuron_forward(xd, wd, y, pos, 1, q, K)
    ext.sort_neuron_forward_nograd(xd, wd, yn, 1, q, K)
    ry, rpos = oracle.sort_neuron_forward(xs, wn, q, K)
    _close(y[:ROWS], ry)
    _close(yn[:ROWS], ry)
    assert np.array_equal(pos[:, :ROWS].cpu().numpy(), rpos)
    eps = np.float32(2.0 / 255)
    xl, xu = (x - eps).contiguous(), (x + eps).contiguous()
    yl, yu = torch.empty_like(y), torch.empty_like(y)
    ext.bound_sort_neuron_forward(xl.to(dev), xu.to(dev), wd, yl, yu, 1, q, K)
    ryl, ryu = oracle.bound_sort_neuron_forward(xl[:ROWS].numpy(), xu[:ROWS].numpy(), wn, q, K)
    _close(yl[:ROWS], ryl)
    _close(yu[:ROWS], ryu)
    assert bool((yl <= yn * (1 + 1e-5)).all()) and bool((yn <= yu * (1 + 1e-5)).all())


@pytest.mark.parametrize("p", [8.0, 64.0])
def test_norm_dist_512x5120x5120(oracle, p):
    """l-p layer forward + backward, B=512, N=M=5120, x ~ N(0,1), followed by the mean shift."""
    from sortnet_amd import ext
    dev = _dev()
    B = 512
    N = M = 5120
    rows = 6
    x, w, gy = _inputs(B, N, M, "randn")
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    y = torch.empty(B, M, 1, device=dev)
    ext.norm_dist_forward(xd, wd, y, 1, p)
    ry = oracle.norm_dist_forward(x[:rows].numpy(), w.numpy(), p)
    _close(y[:rows], ry)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    ext.norm_dist_backward_input_weight(gd, xd, wd, y, gx, gw, 1, p)
    gx2 = torch.empty_like(xd)
    ext.norm_dist_backward_input(gd, xd, wd, y, gx2, 1, p)
    rgx = oracle.norm_dist_backward(gy[:rows].numpy(), x[:rows].numpy(), w.numpy(), ry, p, 1, False)
    _close(gx[:rows], rgx)
    _close(gx2[:rows], rgx)
    # grad_w of a slice of weight rows from the formula in float64 on the device
    ms = slice(1000, 1016)
    d = xd.view(B, 1, N).double() - wd[ms].view(1, -1, N).double()
    u = gd[:, ms].double() * torch.sign(d) * (d.abs() / y[:, ms].double()) ** (p - 1)
    _close(gw[ms], (-u.sum(0)).float())
    out = torch.empty_like(y)
    mean, running = torch.empty(M, device=dev), torch.zeros(M, device=dev)
    ext.mean_shift_forward(y, mean, running, 0.1, out)
    _close(mean, y.mean(dim=(0, 2)))
    _close(out, y - y.mean(dim=(0, 2), keepdim=True))


def test_wide_layers_256x12288x10240():
    """Widest configuration (B=256, 12288 -> 10240 -> 10240): size-independent properties."""
    from sortnet_amd import ext
    dev = _dev()
    B = 256
    g = torch.Generator().manual_seed(0)
    x = torch.rand(B, 12288, generator=g).unsqueeze(-1).contiguous().to(dev)
    eps = 1.0 / 255
    for N, M in ((12288, 10240), (10240, 10240)):
        w = (torch.randn(M, N, generator=g) * N ** -0.5).contiguous().to(dev)
        gy = torch.randn(B, M, 1, generator=g).to(dev)
        y = torch.empty(B, M, 1, device=dev)
        yn = torch.empty_like(y)
        pos = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
        ext.inf_dist_forward(x, w, y, pos, 1)
        ext.inf_dist_forward_nograd(x, w, yn, 1)
        assert torch.equal(y, yn)
        idx = (pos & 0x7FFFFFFF).long().view(B, M)
        dsel = torch.gather(x.view(B, N), 1, idx) - w[torch.arange(M, device=dev).view(1, M), idx]
        assert torch.equal(dsel.abs().clamp(min=1e-10), y.view(B, M))
        assert torch.equal(dsel < 0, pos.view(B, M) < 0)
        # lowest index wins: nothing before the reported position reaches the value
        ref = (x.view(B, 1, N)[:4] - w.view(1, M, N)).abs()
        first = (ref >= y[:4]).float().argmax(dim=-1)
        assert torch.equal(first, idx[:4])
        del ref
        gx, gw = torch.empty_like(x), torch.empty_like(w)
        ext.inf_dist_backward_input_weight(gy, pos, gx, gw, 1)
        tgx, tgw = _scatter_reference(gy, pos, B, N, M, dev)
        _close(gx.view(B, N), tgx)
        _close(gw, tgw)
        ym = torch.empty_like(y)
        ext.masked_inf_dist_forward(x, w, ym, None, 1, 0.3, 3, ext.MASK_FACTORED)
        assert bool((ym <= y).all())
        xl, xu = (x - eps).contiguous(), (x + eps).contiguous()
        yl, yu = torch.empty_like(y), torch.empty_like(y)
        ext.bound_inf_dist_forward_nograd(xl, xu, w, yl, yu, 1)
        assert bool((yl <= y).all()) and bool((y <= yu).all()) and bool((yu - yl <= 2 * eps + 1e-6).all())
        dl, du = torch.empty_like(y), torch.empty_like(y)
        ext.bound_inf_dist_forward_nograd(x, x, w, dl, du, 1)
        assert torch.equal(du, y)
        x = (y - y.mean(dim=0, keepdim=True)).contiguous()
        del w, gw, tgw


def test_index_lists_512x5120x5120():
    """Index-list form at the benchmark size (keep probability 0.3 on both sides).  Every 32-sample sub-batch is
    an ordinary dense problem on the gathered operands x[:, kept inputs] and W[kept outputs][:, kept inputs]:
    the dense entry points (other kernels: vector loads, wide tiles) must give the same l-inf values and
    positions bit for bit, the same l-p values to rel 1e-5, and the scatter backward must match index_put_."""
    from sortnet_amd import ext
    dev = _dev()
    B, N, M = 512, 5120, 5120
    S = B // 32
    _, w, _ = _inputs(B, N, M, "rand")
    wd = w.to(dev)
    cn, cm = ext.mask_count(1, N, 0.3), ext.mask_count(2, M, 0.3)
    ci = ext.sample_index_lists(1, S, 1, N, cn, dev)
    co = ext.sample_index_lists(2, S, 1, M, cm, dev)
    g = torch.Generator().manual_seed(3)
    xc = torch.rand(B, cn, 1, generator=g).to(dev)
    gy = torch.randn(B, cm, 1, generator=g).to(dev)
    y = torch.empty(B, cm, 1, device=dev)
    pos = torch.empty(B, cm, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(xc, wd, y, pos, 1, ci, co)
    yp = torch.empty_like(y)
    ext.norm_dist_forward(xc, wd, yp, 1, 8.0, ci, co)
    for s in (0, 7, S - 1):
        rows = slice(32 * s, 32 * s + 32)
        wsub = wd[co[s, 0].long()][:, ci[s, 0].long()].contiguous()        # (cm, cn)
        xs = xc[rows].contiguous()
        ys = torch.empty(32, cm, 1, device=dev)
        ps = torch.empty(32, cm, 1, device=dev, dtype=torch.int32)
        ext.inf_dist_forward(xs, wsub, ys, ps, 1)
        assert torch.equal(ys, y[rows]) and torch.equal(ps, pos[rows])
        ext.norm_dist_forward(xs, wsub, ys, 1, 8.0)
        _close(yp[rows], ys)
    assert float(y.min()) > 1e-10
    # backward: grad_x[b, n'] += s g, grad_w[co[m'], ci[n']] -= s g through the compact positions
    gx, gw = torch.empty_like(xc), torch.empty_like(wd)
    ext.inf_dist_backward_input_weight(gy, pos, gx, gw, 1, ci, co)
    npos = (pos & 0x7fffffff).long().squeeze(-1)                          # (B, cm) compact input index
    sg = torch.where(pos.squeeze(-1) < 0, -gy.squeeze(-1), gy.squeeze(-1))
    ref_gx = torch.zeros(B, cn, device=dev).index_put_((torch.arange(B, device=dev).unsqueeze(1).expand_as(npos), npos),
                                                       sg, accumulate=True)
    _close(gx.squeeze(-1), ref_gx)
    sub = torch.arange(B, device=dev) // 32
    wrow = co[sub, 0].long()                                              # (B, cm) full output channel
    wcol = torch.gather(ci[sub, 0].long(), 1, npos)                       # (B, cm) full input channel
    ref_gw = torch.zeros(M, N, device=dev).index_put_((wrow, wcol), -sg, accumulate=True)
    _close(gw, ref_gw)

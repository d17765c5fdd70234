#!/usr/bin/env python3
"""Per-entry-point timings of the distance-neuron library at the component configurations
(single layer, fp32): every C-ABI forward/backward op at one shape, with the time per (b, m, n) term
and the fraction of the fp32 vector peak its algorithmic flop count amounts to.

    python bench_ops.py                      # B=512, N=M=5120 (masked / sort / interval / l-p configs)
    python bench_ops.py --shape 128 3072 1024   # the single l-inf layer configuration
"""
import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK = 157.3e12


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--shape", type=int, nargs=3, default=[512, 5120, 5120], metavar=("B", "N", "M"))
    ap.add_argument("--ops", default="linf,mask,bwd,bound,sort,lp,shift,idx")
    ap.add_argument("--reps", type=int, default=5)
    ap.add_argument("--keep", type=float, default=0.3, help="keep probability of the index-list rows")
    ap.add_argument("--data", choices=["config", "unit"], default="config",
                    help="config: inputs ~ U[0,1], weights ~ N(0, 1/N) (the benchmark configurations); unit: weights ~ "
                         "N(0, 1) as the reference initialises them against batch rows that are alike (centred "
                         "activations): the regime of the candidate-table kernels")
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args()
    import torch
    from sortnet_amd import ext, _lib
    dev = torch.device("cuda:0")
    B, N, M = args.shape
    g = torch.Generator().manual_seed(0)
    if args.data == "unit":
        x = (torch.randn(1, N, 1, generator=g) * 0.3 + torch.randn(B, N, 1, generator=g) * 0.1).contiguous().to(dev)
        w = torch.randn(M, N, generator=g).to(dev)
    else:
        x = torch.rand(B, N, 1, generator=g).to(dev)
        w = (torch.randn(M, N, generator=g) * N ** -0.5).to(dev)
    gy = torch.randn(B, M, 1, generator=g).to(dev)
    xn = torch.randn(B, N, 1, generator=g).to(dev)
    xl, xu = (x - 2 / 255).contiguous(), (x + 2 / 255).contiguous()
    y, y2 = torch.empty(B, M, 1, device=dev), torch.empty(B, M, 1, device=dev)
    pos = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
    pos2 = torch.empty_like(pos)
    posK = torch.empty(10, B, M, 1, device=dev, dtype=torch.int32)
    gx, gx2, gw = torch.empty_like(x), torch.empty_like(x), torch.empty_like(w)
    mean = torch.empty(M, device=dev)
    terms = B * N * M
    rows = []

    def t(name, f, flops_per_term=None, nbytes=None):
        f()
        torch.cuda.synchronize()
        # the share of its terms that a forward call formed (below 1: a candidate-table kernel served it)
        share = _lib.last_forward_term_share() if flops_per_term and name.split()[0].endswith(("forward", "forward_nograd", "factored")) else None
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.reps):
            f()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / args.reps
        row = {"op": name, "ms": ms, "fs_per_term": ms * 1e-3 / terms * 1e15}
        if flops_per_term:
            row["tflops"] = flops_per_term * terms / (ms * 1e-3) / 1e12
            row["frac_fp32_peak"] = row["tflops"] * 1e12 / PEAK
        if nbytes:
            row["gb_per_s"] = nbytes / (ms * 1e-3) / 1e9
        if share is not None and share < 1.0:
            row["terms_formed_share"] = share
        rows.append(row)
        if not args.json:
            extra = "  %6.1f TFLOP/s %5.1f%%" % (row["tflops"], 100 * row["frac_fp32_peak"]) if flops_per_term else ""
            extra += "  %7.1f GB/s" % row["gb_per_s"] if nbytes else ""
            extra += "  (from tables: %.1f%% of the terms formed)" % (100 * share) if share is not None and share < 1.0 else ""
            print("%-38s %8.3f ms %7.1f fs/term%s" % (name, ms, row["fs_per_term"], extra), flush=True)

    on = set(args.ops.split(","))
    scat = 4 * (2 * B * M + B * N + M * N)
    if "linf" in on:
        t("inf_dist_forward_nograd", lambda: ext.inf_dist_forward_nograd(x, w, y, 1), 2)
        t("inf_dist_forward (+pos)", lambda: ext.inf_dist_forward(x, w, y, pos, 1), 2)
    if "mask" in on:
        t("masked factored (+pos)", lambda: ext.masked_inf_dist_forward(x, w, y, pos, 1, 0.3, 1, 1), 2)
        t("masked factored nograd", lambda: ext.masked_inf_dist_forward(x, w, y, None, 1, 0.3, 1, 1), 2)
        t("masked term (+pos)", lambda: ext.masked_inf_dist_forward(x, w, y, pos, 1, 0.3, 1, 0), 2)
        t("masked term nograd", lambda: ext.masked_inf_dist_forward(x, w, y, None, 1, 0.3, 1, 0), 2)
    if "bwd" in on:
        ext.inf_dist_forward(x, w, y, pos, 1)
        t("inf_dist_backward_input_weight", lambda: ext.inf_dist_backward_input_weight(gy, pos, gx, gw, 1), None, scat)
        t("inf_dist_backward_input", lambda: ext.inf_dist_backward_input(gy, pos, gx, 1), None, 4 * (2 * B * M + B * N))
    if "bound" in on:
        t("bound_inf_dist_forward_nograd", lambda: ext.bound_inf_dist_forward_nograd(xl, xu, w, y, y2, 1), 6)
        t("bound_inf_dist_forward (+pos)", lambda: ext.bound_inf_dist_forward(xl, xu, w, y, y2, pos, pos2, 1), 6)
        t("bound_inf_dist_backward_input_weight",
          lambda: ext.bound_inf_dist_backward_input_weight(gy, gy, pos, pos2, gx, gx2, gw, 1), None,
          4 * (4 * B * M + 2 * B * N + M * N))
    if "sort" in on:
        t("sort_neuron_forward_nograd K=10", lambda: ext.sort_neuron_forward_nograd(x, w, y, 1, 0.3, 10), 2)
        t("sort_neuron_forward K=10", lambda: ext.sort_neuron_forward(x, w, y, posK, 1, 0.3, 10), 2)
        t("bound_sort_neuron_forward K=10", lambda: ext.bound_sort_neuron_forward(xl, xu, w, y, y2, 1, 0.3, 10), 6)
        t("sort_neuron_backward_input_weight K=10",
          lambda: ext.sort_neuron_backward_input_weight(gy, posK, gx, gw, 1, 0.3, 10), None,
          4 * (11 * B * M + B * N + M * N))
    if "lp" in on:
        for p, ff, fb in ((8.0, 5, 9), (24.0, 3, 5), (64.0, 3, 5), (256.0, 3, 5)):
            t("norm_dist_forward p=%g" % p, lambda: ext.norm_dist_forward(xn, w, y, 1, p), ff)
            t("norm_dist_backward_input_weight p=%g" % p,
              lambda: ext.norm_dist_backward_input_weight(gy, xn, w, y, gx, gw, 1, p), fb)
            t("norm_dist_backward_input p=%g" % p, lambda: ext.norm_dist_backward_input(gy, xn, w, y, gx, 1, p), fb / 2)
        if not args.json:
            print("  (general p: the rate counts all B*M*N terms; the candidate-table kernels evaluate marked inputs only,"
                  " so it can exceed the peak)", flush=True)
    if "idx" in on:
        # index-list ("dropout") form: every 32-sample sub-batch keeps its own ~q share of the inputs and outputs
        qk = args.keep
        S = (B + 31) // 32
        cn, cm = ext.mask_count(1, N, qk), ext.mask_count(2, M, qk)
        ci = ext.sample_index_lists(1, S, 1, N, cn, dev)
        co = ext.sample_index_lists(2, S, 1, M, cm, dev)
        xc = torch.rand(B, cn, 1, generator=g).to(dev)
        gyc = torch.randn(B, cm, 1, generator=g).to(dev)
        yc = torch.empty(B, cm, 1, device=dev)
        posc = torch.empty(B, cm, 1, device=dev, dtype=torch.int32)
        gxc = torch.empty_like(xc)
        sub = B * cn * cm
        scale = terms / sub          # the helper divides by the dense term count
        t("index lists: %d of %d in, %d of %d out" % (cn, N, cm, M), lambda: None)
        rows.pop()
        t("  sample_index_lists (both)", lambda: (ext.sample_index_lists(1, S, 1, N, cn, dev),
                                                   ext.sample_index_lists(2, S, 1, M, cm, dev)))
        t("  inf_dist_forward (+pos, lists)", lambda: ext.inf_dist_forward(xc, w, yc, posc, 1, ci, co), 2 / scale)
        t("  inf_dist_backward_input_weight (lists)",
          lambda: ext.inf_dist_backward_input_weight(gyc, posc, gxc, gw, 1, ci, co))
        t("  norm_dist_forward p=8 (lists)", lambda: ext.norm_dist_forward(xc, w, yc, 1, 8.0, ci, co), 5 / scale)
        t("  norm_dist_backward_input p=8 (lists)",
          lambda: ext.norm_dist_backward_input(gyc, xc, w, yc, gxc, 1, 8.0, ci, co), 4.5 / scale)
        t("  norm_dist_backward_input_weight p=8 (lists)",
          lambda: ext.norm_dist_backward_input_weight(gyc, xc, w, yc, gxc, gw, 1, 8.0, ci, co), 9 / scale)
        for p in (24.0, 256.0):
            t("  norm_dist_forward p=%g (lists)" % p, lambda: ext.norm_dist_forward(xc, w, yc, 1, p, ci, co), 3 / scale)
            t("  norm_dist_backward_input_weight p=%g (lists)" % p,
              lambda: ext.norm_dist_backward_input_weight(gyc, xc, w, yc, gxc, gw, 1, p, ci, co), 5 / scale)
        meanc = torch.empty(M, device=dev)
        t("  mean_shift_index_forward (lists)", lambda: ext.mean_shift_index_forward(yc, co, M, meanc, None, 0.1, gyc),
          None, 4 * (3 * B * cm))
    if "shift" in on:
        t("mean_shift_forward", lambda: ext.mean_shift_forward(y, mean, None, 0.1, y2), None, 4 * (3 * B * M))
    if args.json:
        print(json.dumps({"shape": {"B": B, "N": N, "M": M}, "rows": rows}))


if __name__ == "__main__":
    main()

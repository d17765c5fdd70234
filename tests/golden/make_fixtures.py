#!/usr/bin/env python3
"""Writes tests/golden/vectors.json: small known-answer vectors for the distance-neuron ops.

Every expected value is computed here from first principles in pure Python / numpy (sequential
scans in float32 for the bit-exact sets, float64 closed forms for the tolerance sets, Python
integers for the counter RNG) - neither the CPU oracle nor the GPU library is imported, so the
fixture pins both of them to the written definition of each op:

* l-inf forward (core/cuda/inf_dist_cuda.cu:135-211): strict `>` scan from (1e-10, index 0),
  pos = lowest arg-max index | sign bit of x - w;
* interval bounds (core/cuda/bound_inf_dist_cuda.cu:141-237): repair of inverted intervals, t1 = w - xL,
  t2 = xU - w, lower position starts at the 0xffffffff sentinel;
* sort neuron (core/cuda/sort_neuron.cu:73-97, 176-209): ordered insertion, geometric weights;
* l-p distance (core/cuda/norm_dist_cuda.cu:61-71, 251-266): value and gradients in float64;
* the counter RNG of the masked neuron and of the index-list sampler (defined by this build).

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import json
import os

import numpy as np

F = np.float32
EPS = F(1e-10)
SIGN = 0x80000000
M32 = 0xFFFFFFFF


def rng_inputs(seed, shape, kind):
    r = np.random.default_rng(seed)
    a = r.random(shape) if kind == "rand" else r.standard_normal(shape)
    return np.asarray(a, dtype=np.float32)


# ---------------------------------------------------------------- counter RNG in Python integers
def mix(h):
    h ^= h >> 16
    h = (h * 0x21F0AAAD) & M32
    h ^= h >> 15
    h = (h * 0x735A2D97) & M32
    h ^= h >> 15
    return h


def row_key(seed, stream, row):
    return mix(((seed ^ ((stream * 0x9E3779B9) & M32)) + row) & M32)


def word(key, col):
    return mix((key + (col + 1) * 0x85EBCA6B) & M32)


def t8_of(q):       # q arrives as a float32 at the library boundary
    return int(np.floor(np.float64(np.float32(q)) * 256.0 + 0.5))


def t16_of(q):
    return int(np.floor(np.sqrt(np.float64(np.float32(q))) * 65536.0 + 0.5))


def keep_term(seed, o, n, q):
    t8 = t8_of(q)
    return ((word(row_key(seed, 0, o), n >> 2) >> (8 * (n & 3))) & 0xFF) < t8


def keep_factored(seed, xrow, wrow, n, q):
    t16 = t16_of(q)
    return (word(row_key(seed, 1, xrow), n) >> 16) < t16 and (word(row_key(seed, 2, wrow), n) >> 16) < t16


# ---------------------------------------------------------------- ops, one output at a time
def linf(xr, wr, keep=None):
    best, pos = EPS, 0
    for n in range(len(xr)):
        if keep is not None and not keep(n):
            continue
        d = F(xr[n] - wr[n])
        v = F(abs(d))
        if v > best:
            best, pos = v, n | (SIGN if d < 0 else 0)
    return float(best), pos


def bound(xl, xu, wr):
    lo, hi, pl, pu = F(-1e-10), EPS, M32, 0
    for n in range(len(wr)):
        l, u = F(xl[n]), F(xu[n])
        if l > u:
            l = u = F(F(l + u) * F(0.5))
        t1, t2 = F(wr[n] - l), F(u - wr[n])
        flag = 0 if t1 <= t2 else SIGN
        mn, mx = min(t1, t2), max(t1, t2)
        if mn < lo:
            lo, pl = mn, n | flag
        if mx > hi:
            hi, pu = mx, n | flag
    return float(F(-lo)), float(hi), pl, pu


def sort_neuron(xr, wr, q, K):
    res, idx = [F(0)] * K, [0] * K          # ascending, res[K-1] largest
    for n in range(len(xr)):
        d = F(xr[n] - wr[n])
        v = F(abs(d))
        if not v > res[0]:
            continue
        p = n | (SIGN if d < 0 else 0)
        k = 0
        while k + 1 < K and v >= res[k + 1]:   # equal values: the later input ranks higher
            res[k], idx[k] = res[k + 1], idx[k + 1]
            k += 1
        res[k], idx[k] = v, p
    c, ans = 1.0, 1e-10
    for k in range(K - 1, -1, -1):
        ans += float(res[k]) * c * q
        c *= 1.0 - q
    return ans / (1.0 - c), idx[::-1]


def lp_forward(x, w, p):
    d = np.abs(x[:, None, :].astype(np.float64) - w[None].astype(np.float64))
    return (d ** p).sum(-1) ** (1.0 / p)


def lp_backward(g, x, w, y, p):
    d = x[:, None, :].astype(np.float64) - w[None].astype(np.float64)
    u = g[:, :, None] * np.sign(d) * (np.abs(d) / y[:, :, None]) ** (p - 1)
    return u.sum(1), -u.sum(0)


def sample_lists(seed, S, G, C, q):
    thr = int(np.floor(np.float64(np.float32(q)) * 4294967296.0 + 0.5))
    k3 = row_key(seed, 3, 0)
    count = sum(1 for c in range(C) if word(k3, c) < thr)
    lists = []
    for r in range(S * G):
        kr = row_key(seed, 4, r)
        keys = sorted(((word(kr, c) << 16) | c) for c in range(C))[:count]
        lists.append(sorted(k & 0xFFFF for k in keys))
    return count, np.array(lists, dtype=np.int64).reshape(S, G, count)


def main():
    out = {}
    B, N, M = 5, 24, 7
    x = rng_inputs(11, (B, N), "rand")
    w = rng_inputs(12, (M, N), "randn") * F(0.5)
    # exact ties and an all-zero row
    w[0, :] = x[0, :]
    w[1, 3], w[1, 9], w[1, 17] = x[1, 3] + F(2), x[1, 9] - F(2), x[1, 17] + F(2)
    g = rng_inputs(13, (B, M), "randn")

    ys, ps = zip(*[linf(x[b], w[m]) for b in range(B) for m in range(M)])
    out["linf"] = {"x": x.tolist(), "w": w.tolist(), "y": np.array(ys, np.float32).reshape(B, M).tolist(),
                   "pos": np.array(ps, np.int64).reshape(B, M).tolist()}

    seed, q = 77, 0.3
    for mode, name in ((0, "masked_term"), (1, "masked_factored")):
        ys, ps = [], []
        for b in range(B):
            for m in range(M):
                keep = (lambda n, o=b * M + m: keep_term(seed, o, n, q)) if mode == 0 else \
                       (lambda n, b=b, m=m: keep_factored(seed, b, m, n, q))
                yv, pv = linf(x[b], w[m], keep)
                ys.append(yv), ps.append(pv)
        out[name] = {"seed": seed, "q": q, "y": np.array(ys, np.float32).reshape(B, M).tolist(),
                     "pos": np.array(ps, np.int64).reshape(B, M).tolist()}

    xl = (x - F(0.05)).astype(np.float32)
    xu = (x + F(0.05)).astype(np.float32)
    xl[2, 5], xu[2, 5] = F(0.9), F(0.1)                  # inverted interval: repaired to the midpoint
    w[3, :] = ((xl[3] + xu[3]) * F(0.5)).astype(np.float32)   # inside every interval of sample 3
    res = [bound(xl[b], xu[b], w[m]) for b in range(B) for m in range(M)]
    out["bound"] = {"xl": xl.tolist(), "xu": xu.tolist(), "w": w.tolist(),
                    "yl": np.array([r[0] for r in res], np.float32).reshape(B, M).tolist(),
                    "yu": np.array([r[1] for r in res], np.float32).reshape(B, M).tolist(),
                    "pl": np.array([r[2] for r in res], np.int64).reshape(B, M).tolist(),
                    "pu": np.array([r[3] for r in res], np.int64).reshape(B, M).tolist()}

    K, qs = 4, 0.4
    xs = np.round(x * 4) / 4                               # coarse grid: many equal magnitudes
    ws = np.round(w * 2) / 2
    res = [sort_neuron(xs[b].astype(np.float32), ws[m].astype(np.float32), qs, K) for b in range(B) for m in range(M)]
    out["sort"] = {"x": xs.tolist(), "w": ws.tolist(), "q": qs, "K": K,
                   "y": np.array([r[0] for r in res]).reshape(B, M).tolist(),
                   "pos": np.array([r[1] for r in res], np.int64).reshape(B, M, K).transpose(2, 0, 1).tolist()}

    xn = rng_inputs(14, (B, N), "randn")
    out["lp"] = {"x": xn.tolist(), "w": w.tolist(), "g": g.tolist(), "cases": []}
    for p in (3.0, 8.0, 20.0, 9.5, 4.0, 5.0, 6.0, 9.0, 1.5):
        y = lp_forward(xn, w, p)
        gx, gw = lp_backward(g.astype(np.float64), xn, w, y, p)
        out["lp"]["cases"].append({"p": p, "y": y.tolist(), "gx": gx.tolist(), "gw": gw.tolist()})

    out["rng"] = {"words": [[s, st, r, c, word(row_key(s, st, r), c)] for s, st, r, c in
                            ((0, 0, 0, 0), (1, 0, 0, 0), (77, 1, 5, 9), (0xDEADBEEF, 2, 123456, 4095),
                             (M32, 4, M32, M32), (12345, 3, 0, 17))],
                  "t8": [[qq, t8_of(qq)] for qq in (0.0, 0.3, 0.5, 1.0)],
                  "t16": [[qq, t16_of(qq)] for qq in (0.0, 0.3, 0.5, 1.0)]}
    samplers = []
    for sd, S, G, C, qq in ((5, 3, 1, 40, 0.3), (9, 2, 2, 33, 0.75), (1, 1, 1, 16, 1.0)):
        count, lists = sample_lists(sd, S, G, C, qq)
        samplers.append({"seed": sd, "S": S, "G": G, "C": C, "q": qq, "count": count, "lists": lists.tolist()})
    out["sampler"] = samplers

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.json")
    with open(path, "w") as f:
        json.dump(out, f)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()

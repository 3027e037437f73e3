"""The oracle's sampler functions against independent statements of what they compute, and the library's host-side
sampler functions against the oracle (no GPU here).

top_tokens (topk.cuh): numpy's lexsort on (key descending, id ascending) with the order-preserving key written out in
numpy; rows of equal logits, signed zeros, infinities and NaNs; bias and penalties as numpy float32 arithmetic.
make_dist (session.cpp:41-75): numpy's vectorised softmax and cumulative cut; the limiting cases.
accept_sampled (session.cpp:574-613): what speculative sampling is for - the first token of a window is distributed as
the target distribution p whatever the draft distribution q was - measured exactly over a grid of the uniforms."""
import ctypes as C

import numpy as np
import pytest

import fnx_gpu
import oracle_lib as ol


def np_key(x):
    u = x.view(np.uint32).astype(np.uint64)
    return np.where(u & 0x80000000, (~u) & 0xFFFFFFFF, u | 0x80000000).astype(np.int64)


def np_top64(row, v0=0):
    order = np.lexsort((np.arange(row.size), -np_key(row)))[:64]
    return row[order], order.astype(np.int32) + v0


def o_top_tokens(oracle, logits, v0=0, pen=None, par=None, bias=None):
    """pen: per row list of (token, count); par: per row (repeat, freq, present); bias: per row list of (token, value)"""
    T, n = logits.shape
    L = np.ascontiguousarray(logits, dtype=np.float32).copy()
    a = pack_lists(T, pen, par, bias)
    ov, oi = np.zeros((T, 64), np.float32), np.zeros((T, 64), np.int32)
    err = oracle.lib.fnx_o_top_tokens(ol.ptr(L), n, T, v0, ol.ptr(a["pen_tok"]), ol.ptr(a["pen_cnt"]), ol.ptr(a["pen_n"]), a["stride"], ol.ptr(a["par"]),
                                      ol.ptr(a["bias_tok"]), ol.ptr(a["bias_val"]), ol.ptr(a["bias_off"]), ol.ptr(a["bias_n"]), ol.ptr(ov), ol.ptr(oi))
    return ov, oi, L, err


def pack_lists(T, pen, par, bias):
    pen = pen or [[] for _ in range(T)]
    bias = bias or [[] for _ in range(T)]
    stride = max(1, max(len(p) for p in pen))
    a = dict(stride=stride, pen_tok=np.zeros((T, stride), np.int32), pen_cnt=np.zeros((T, stride), np.int32), pen_n=np.array([len(p) for p in pen], np.int32),
             par=np.array(par if par else [(1.0, 0.0, 0.0)] * T, np.float32).reshape(T, 3), bias_n=np.array([len(b) for b in bias], np.int32))
    for t, p in enumerate(pen):
        for i, (tok, cnt) in enumerate(p):
            a["pen_tok"][t, i], a["pen_cnt"][t, i] = tok, cnt
    a["bias_off"] = np.concatenate([[0], np.cumsum(a["bias_n"])[:-1]]).astype(np.int32)
    flat = [e for b in bias for e in b]
    a["bias_tok"] = np.array([e[0] for e in flat] or [0], np.int32)
    a["bias_val"] = np.array([e[1] for e in flat] or [0], np.float32)
    return a


def test_top_tokens_equals_numpy_lexsort(oracle):
    rng = np.random.default_rng(2)
    for n in (64, 65, 1000, 5000):
        x = rng.standard_normal((3, n)).astype(np.float32)
        x[1, rng.integers(0, n, n // 2)] = 1.5        # wide ties inside the candidates
        x[2] = np.round(x[2] * 2) / 2                 # few distinct values: ties at the threshold
        ov, oi, L, err = o_top_tokens(oracle, x, v0=7)
        assert err == 0 and np.array_equal(L, x)
        for t in range(3):
            wv, wi = np_top64(x[t], 7)
            assert np.array_equal(oi[t], wi) and np.array_equal(ov[t].view(np.uint32), wv.view(np.uint32))
    eq = np.full((1, 300), -2.25, np.float32)       # a row of equal logits: the 64 lowest ids
    assert np.array_equal(o_top_tokens(oracle, eq)[1][0], np.arange(64))
    z = np.zeros((1, 128), np.float32)
    z[0, 63:] = -0.0                                  # +0 ranks above -0 (the key is of the bits)
    z[0, 100] = 0.0
    assert np.array_equal(o_top_tokens(oracle, z)[1][0], list(range(63)) + [100])
    bad = rng.standard_normal((2, 200)).astype(np.float32)
    bad[0, 5], bad[1, 7], bad[1, 9] = np.inf, np.nan, -np.inf
    ov, oi, _, err = o_top_tokens(oracle, bad)
    assert err == 16 and oi[0, 0] == 5 and oi[1, 0] == 7, "+inf and a positive NaN's bits rank first"
    assert 9 not in oi[1]


def test_bias_and_penalties_equal_numpy_float32(oracle):
    rng = np.random.default_rng(3)
    n, T, v0 = 400, 4, 1000
    x = rng.standard_normal((T, n)).astype(np.float32) * 3
    pen = [[(v0 + int(t), int(c)) for t, c in zip(rng.choice(n, 40, replace=False), rng.integers(0, 4, 40))] + [(5, 2), (v0 + n, 1)] for _ in range(T)]
    par = [(1.3, 0.1, 0.2), (0.8, 0.0, 0.5), (1.0, 0.25, 0.0), (2.0, 0.5, 0.5)]
    bias = [[(v0 + int(t), float(b)) for t, b in zip(rng.choice(n, 10, replace=False), rng.standard_normal(10) * 5)] + [(3, 9.0)] for _ in range(T)]
    want = x.copy()
    f32 = np.float32
    for t in range(T):
        for tok, b in bias[t]:
            if 0 <= tok - v0 < n:
                want[t, tok - v0] = f32(want[t, tok - v0] + f32(b))
        for tok, c in pen[t]:
            j = tok - v0
            if not (0 <= j < n) or c <= 0:
                continue
            l = want[t, j]
            l = f32(l * f32(par[t][0])) if l <= 0 else f32(l / f32(par[t][0]))
            want[t, j] = f32(f32(l - f32(f32(c) * f32(par[t][1]))) - f32(par[t][2]))
    ov, oi, L, err = o_top_tokens(oracle, x, v0=v0, pen=pen, par=par, bias=bias)
    assert np.array_equal(L.view(np.uint32), want.view(np.uint32)), "the row is changed in place: bias first, then the penalties"
    for t in range(T):
        wv, wi = np_top64(want[t], v0)
        assert np.array_equal(oi[t], wi) and np.array_equal(ov[t], wv)
    row = x[0].copy()
    k = len(pen[0])
    packed = np.array([k] + [tok - v0 for tok, _ in pen[0]] + [c for _, c in pen[0]], np.int32)
    oracle.lib.fnx_o_penalize_row(ol.ptr(row), n, ol.ptr(packed), ol.ptr(np.array(par[0], np.float32)))
    only_pen = x[0].copy()
    for tok, c in pen[0]:
        j = tok - v0
        if 0 <= j < n and c > 0:
            l = only_pen[j]
            l = f32(l * f32(par[0][0])) if l <= 0 else f32(l / f32(par[0][0]))
            only_pen[j] = f32(f32(l - f32(f32(c) * f32(par[0][1]))) - f32(par[0][2]))
    assert np.array_equal(row, only_pen)


def o_dist(oracle, cv, ci, temperature=1.0, top_p=1.0, min_p=0.0, top_k=0):
    ids, p = np.zeros(len(cv), np.int32), np.zeros(len(cv), np.float64)
    k = oracle.lib.fnx_o_make_dist(ol.ptr(cv), ol.ptr(ci), len(cv), temperature, top_p, min_p, top_k, ol.ptr(ids), ol.ptr(p))
    return ids[:k], p[:k]


def np_dist(cv, ci, temperature=1.0, top_p=1.0, min_p=0.0, top_k=0):
    v = cv.astype(np.float64)
    k = len(v) if top_k <= 0 or top_k > len(v) else top_k
    keep = k
    if np.float32(top_p) < 1:
        sm = np.exp(v[:k] - v[0])
        cum = np.cumsum(sm / sm.sum())
        hit = np.nonzero(cum >= np.float64(np.float32(top_p)))[0]
        keep = int(hit[0]) + 1 if hit.size else k
    if np.float32(min_p) > 0:
        below = np.nonzero(cv[1:keep] < np.float32(cv[0] + np.log(np.float32(min_p))))[0]
        keep = int(below[0]) + 1 if below.size else keep
    inv_t = 1.0 / np.float64(np.float32(temperature))
    e = np.exp(v[:keep] * inv_t - v[0] * inv_t)
    return ci[:keep], e / e.sum()


def test_make_dist_equals_numpy_and_limits(oracle):
    rng = np.random.default_rng(4)
    for _ in range(200):
        m = int(rng.integers(1, 65))
        cv = np.sort(rng.standard_normal(m).astype(np.float32) * 3)[::-1].copy()
        ci = rng.permutation(1000)[:m].astype(np.int32)
        kw = dict(temperature=float(rng.choice([0.3, 0.7, 1.0, 1.5])), top_p=float(rng.choice([1.0, 0.95, 0.5, 0.1])),
                  min_p=float(rng.choice([0.0, 0.05, 0.3])), top_k=int(rng.choice([0, 1, 5, 40, 100])))
        ids, p = o_dist(oracle, cv, ci, **kw)
        wi, wp = np_dist(cv, ci, **kw)
        assert np.array_equal(ids, wi) and np.allclose(p, wp, rtol=1e-12, atol=0) and abs(p.sum() - 1) < 1e-12
    cv, ci = np.array([2.0, 1.0, 0.0, -1.0], np.float32), np.arange(4, dtype=np.int32)
    ids, p = o_dist(oracle, cv, ci)
    assert np.allclose(p, np.exp(cv.astype(np.float64)) / np.exp(cv.astype(np.float64)).sum(), rtol=1e-15)   # plain softmax
    assert len(o_dist(oracle, cv, ci, top_k=1)[0]) == 1 and len(o_dist(oracle, cv, ci, top_p=1e-6)[0]) == 1
    assert np.allclose(o_dist(oracle, cv, ci, temperature=1e-3)[1], [1, 0, 0, 0], atol=1e-300)
    assert len(o_dist(oracle, cv, ci, min_p=float(np.exp(-1.5)))[0]) == 2, "min_p is a threshold on the logit: ln(min_p) below the best"
    assert [oracle.lib.fnx_o_draw(ol.ptr(ci), ol.ptr(p), 4, u) for u in (0.0, float(p[0]) - 1e-9, float(p[0]) + 1e-9, 0.999999, 1.0)] == [0, 0, 1, 3, 3]


def o_accept(oracle, cv, ci, rows, u, q=None, **kw):
    T, m = cv.shape
    kw = dict(dict(temperature=1.0, top_p=1.0, min_p=0.0, top_k=0), **kw)
    qi = qp = qn = None
    stride = 1
    if q is not None:
        stride = max(1, max(len(d[0]) for d in q))
        qi, qp, qn = np.zeros((len(q), stride), np.int32), np.zeros((len(q), stride), np.float64), np.array([len(d[0]) for d in q], np.int32)
        for j, (ids, p) in enumerate(q):
            qi[j, :len(ids)], qp[j, :len(ids)] = ids, p
    o, used = np.zeros(T, np.int32), C.c_int()
    u = np.ascontiguousarray(u, np.float64)
    n = oracle.lib.fnx_o_accept_sampled(ol.ptr(cv), ol.ptr(ci), m, T, ol.ptr(np.asarray(rows, np.int32)), kw["temperature"], kw["top_p"], kw["min_p"],
                                        kw["top_k"], ol.ptr(qi), ol.ptr(qp), ol.ptr(qn), stride, ol.ptr(u), ol.ptr(o), C.byref(used))
    return n, list(o[:n]), used.value


def test_speculative_sampling_keeps_the_target_distribution(oracle):
    # a window of two rows, a vocabulary of five: row 0's token over a fine grid of (u_accept, u_draw) has the measure p_0,
    # for a drafted distribution q and for a fixed draft alike
    cv = np.array([[1.2, 0.7, 0.1, -0.4, -1.0], [0.3, 0.2, 0.1, 0.0, -0.1]], np.float32)
    ci = np.array([[3, 1, 4, 0, 2], [0, 1, 2, 3, 4]], np.int32)
    ids, p = o_dist(oracle, cv[0], ci[0])
    target = dict(zip(ids.tolist(), p.tolist()))
    G = 400
    grid = (np.arange(G) + 0.5) / G
    q_ids, q_p = np.array([1, 2, 3], np.int32), np.array([0.6, 0.3, 0.1])
    for q in ([(q_ids, q_p)], None):
        mass = {t: 0.0 for t in range(5)}
        drafts = [(int(t), float(w)) for t, w in zip(q_ids, q_p)] if q else [(1, 1.0)]
        for draft, wq in drafts:   # the draft itself is drawn from q
            for ua in grid:
                # row 0's token does not depend on u_draw when the draft stands: one call covers the column
                n, o, used = o_accept(oracle, cv, ci, [9, draft], [ua, 0.5, 0.5], q=q)
                if n == 2:
                    assert o[0] == draft and used == 2
                    mass[draft] += wq / G
                    continue
                for ud in grid[::8]:
                    n, o, used = o_accept(oracle, cv, ci, [9, draft], [ua, ud], q=q)
                    assert n == 1 and used == 2
                    mass[o[0]] += wq / G / len(grid[::8])
        for t in range(5):
            assert abs(mass[t] - target[t]) < 0.02, (q is not None, t, mass[t], target[t])
    # a fixed draft stands with probability p(draft); when it falls, the token is never the draft
    n, o, _ = o_accept(oracle, cv, ci, [9, 1], [target[1] - 1e-9, 0.3])
    assert n == 2 and o[0] == 1
    n, o, _ = o_accept(oracle, cv, ci, [9, 1], [target[1] + 1e-9, 0.3])
    assert n == 1 and o[0] != 1
    # every draft standing: one more token from the last row, T tokens in all, T uniforms
    n, o, used = o_accept(oracle, cv, ci, [9, 3], [0.0, 0.0])
    assert (n, o, used) == (2, [3, 0], 2)
    # a window of one row is a plain draw
    assert o_accept(oracle, cv[:1], ci[:1], [9], [0.0]) == (1, [3], 1)


def test_library_host_sampler_equals_oracle(oracle):
    pkg = fnx_gpu.package()
    lib = pkg.lib()
    rng = np.random.default_rng(6)
    for _ in range(300):
        T, m = int(rng.integers(1, 17)), int(rng.integers(2, 65))
        cv = -np.sort(-rng.standard_normal((T, m)).astype(np.float32) * 2, axis=1)
        ci = np.stack([rng.permutation(50)[:m] if m <= 50 else rng.permutation(100)[:m] for _ in range(T)]).astype(np.int32)
        kw = dict(temperature=float(rng.choice([0.5, 1.0, 1.3])), top_p=float(rng.choice([1.0, 0.9, 0.6])), min_p=float(rng.choice([0.0, 0.1])),
                  top_k=int(rng.choice([0, 3, 20])))
        s = pkg.Sampling(kw["temperature"], kw["top_p"], kw["min_p"], kw["top_k"])
        ids, p = np.zeros(m, np.int32), np.zeros(m, np.float64)
        k = lib.fnx_make_dist(cv[0].ctypes.data, ci[0].ctypes.data, m, C.byref(s), ids.ctypes.data, p.ctypes.data)
        wi, wp = o_dist(oracle, cv[0], ci[0], **kw)
        assert k == len(wi) and np.array_equal(ids[:k], wi) and np.array_equal(p[:k], wp)
        u1 = float(rng.random())
        assert lib.fnx_draw(ids.ctypes.data, p.ctypes.data, k, u1) == oracle.lib.fnx_o_draw(ol.ptr(wi), ol.ptr(wp), k, u1)
        rows = np.concatenate([[0], [ci[j, int(rng.integers(0, min(3, m)))] for j in range(T - 1)]]).astype(np.int32)
        q = None
        if T > 1 and rng.random() < 0.5:
            q = []
            for j in range(T - 1):
                qn = int(rng.integers(0, 5))
                qi = np.unique(np.concatenate([[rows[j + 1]], rng.integers(0, 100, qn)])).astype(np.int32) if qn else np.zeros(0, np.int32)
                qp = rng.random(len(qi)) + 0.05
                q.append((qi, qp / qp.sum() if len(qi) else qp))
        u = rng.random(T + 1)
        want = o_accept(oracle, cv, ci, rows, u, q=q, **kw)
        qi = qp = qn = None
        stride = 1
        if q is not None:
            stride = max(1, max(len(d[0]) for d in q))
            qi, qp, qn = np.zeros((T - 1, stride), np.int32), np.zeros((T - 1, stride), np.float64), np.array([len(d[0]) for d in q], np.int32)
            for j, (a, b) in enumerate(q):
                qi[j, :len(a)], qp[j, :len(a)] = a, b
        o, used = np.zeros(T, np.int32), C.c_int()
        n = lib.fnx_accept_sampled(cv.ctypes.data, ci.ctypes.data, m, T, rows.ctypes.data, C.byref(s), ol.ptr(qi), ol.ptr(qp), ol.ptr(qn), stride,
                                   u.ctypes.data, len(u), o.ctypes.data, C.byref(used))
        assert (n, list(o[:n]), used.value) == want
    s = pkg.Sampling(0.0, 1.0, 0.0, 0)
    assert lib.fnx_make_dist(cv[0].ctypes.data, ci[0].ctypes.data, m, C.byref(s), ids.ctypes.data, p.ctypes.data) == -1 and b"temperature" in lib.fnx_last_error()
    s = pkg.Sampling(1.0, 1.0, 0.0, 0)
    assert lib.fnx_accept_sampled(cv.ctypes.data, ci.ctypes.data, m, T, rows.ctypes.data, C.byref(s), None, None, None, 1, u.ctypes.data, 0, o.ctypes.data,
                                  C.byref(used)) == -1 and b"uniforms" in lib.fnx_last_error()

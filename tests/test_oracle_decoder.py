"""Pins for the oracle's norm / dense / attention / decoder functions: numpy f64 statements of the same mathematics and
invariants a wrong sign, index or transposition would break."""
import numpy as np

import oracle_lib as ol
import tiny_decoder as td

ROPE = td.RopeO(1e7, 0, 0.0, 0.0, 1.0, 1.0)


def test_rms_norm(oracle):
    rng = np.random.default_rng(1)
    x, w = rng.standard_normal((5, 512)).astype(np.float32), rng.standard_normal(512).astype(np.float32)
    y = np.zeros_like(x)
    oracle.lib.fnx_o_rms_norm_rows(ol.ptr(x), ol.ptr(w), ol.ptr(y), 5, 512, 1e-6)
    want = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
    assert np.allclose(y, want, rtol=3e-7, atol=0)


def q8_0(oracle, w):
    rows, cols = w.shape
    q, d = np.zeros((rows, cols), dtype=np.int8), np.zeros((rows, cols // 32), dtype=np.uint16)
    oracle.lib.fnx_o_quantize_q8_0_split(ol.ptr(w), rows, cols, ol.ptr(q), ol.ptr(d))
    return q, d


def test_q8_0_split_and_gemv(oracle):
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((37, 1024)) * 0.05).astype(np.float32)
    w[3, :32] = 0
    q, d = q8_0(oracle, w)
    blocks = w.reshape(37, 32, 32)
    dd = np.abs(blocks).max(axis=2) / np.float32(127.0)
    assert np.array_equal(d.view(np.float16), dd.astype(np.float16))
    with np.errstate(divide="ignore", invalid="ignore"):
        want_q = np.where(dd[:, :, None] > 0, blocks * (np.float32(1.0) / dd[:, :, None]), 0)
    want_q = np.sign(want_q) * np.floor(np.abs(want_q) + 0.5)   # roundf: halves away from zero
    assert np.array_equal(q.reshape(37, 32, 32), want_q.astype(np.int8))
    x = rng.standard_normal((3, 1024)).astype(np.float32)
    yq = oracle.quantize_q8_1(x)
    out = np.zeros((3, 37), dtype=np.float32)
    oracle.lib.fnx_o_q8s_gemv(ol.ptr(q), ol.ptr(d), 37, 1024, ol.ptr(yq), ol.ptr(out), 37, 3)
    yb = yq.reshape(3, 32, 36)
    xd = yb[:, :, :2].copy().view(np.float16).astype(np.float64)[:, :, 0]
    xq = yb[:, :, 4:].view(np.int8).astype(np.int64)
    sumi = np.einsum("rbj,tbj->trb", q.reshape(37, 32, 32).astype(np.int64), xq)
    want = (sumi * d.view(np.float16).astype(np.float64)[None] * xd[:, None, :]).sum(axis=2)
    assert np.allclose(out, want, rtol=1e-5, atol=1e-6)


def prep(oracle, qg, k, v, qn, kn, kc, vc, nq, nkv, pos0, rope=ROPE, eps=1e-6):
    qg, k = qg.copy(), k.copy()
    oracle.lib.fnx_o_attn_prep_append(ol.ptr(qg), ol.ptr(k), ol.ptr(v), ol.ptr(qn), ol.ptr(kn), ol.ptr(kc), ol.ptr(vc), nq, nkv, 256, 64, qg.shape[0],
                                      pos0, eps, C_byref(rope))
    return qg, k


def C_byref(x):
    import ctypes
    return ctypes.cast(ctypes.pointer(x), ctypes.c_void_p)


def test_attn_prep_append(oracle):
    rng = np.random.default_rng(3)
    nq, nkv, T, pos0 = 4, 2, 3, 5
    qg = rng.standard_normal((T, nq, 512)).astype(np.float32)
    k, v = rng.standard_normal((T, nkv, 256)).astype(np.float32), rng.standard_normal((T, nkv, 256)).astype(np.float32)
    qn, kn = (1 + 0.1 * rng.standard_normal(256)).astype(np.float32), (1 + 0.1 * rng.standard_normal(256)).astype(np.float32)
    kc, vc = np.zeros((16, nkv, 256), dtype=np.uint16), np.zeros((16, nkv, 256), dtype=np.uint16)
    q2, k2 = prep(oracle, qg, k, v, qn, kn, kc, vc, nq, nkv, pos0)

    def want(x, w, pos):
        x = x.astype(np.float64)
        y = x / np.sqrt((x ** 2).mean() + 1e-6) * w
        i = np.arange(32)
        th = pos * (1e7 ** (-2.0 * i / 64))
        x0, x1 = y[:32].copy(), y[32:64].copy()
        y[:32], y[32:64] = x0 * np.cos(th) - x1 * np.sin(th), x0 * np.sin(th) + x1 * np.cos(th)
        return y

    for t in range(T):
        for h in range(nq):
            assert np.allclose(q2[t, h, :256], want(qg[t, h, :256], qn, pos0 + t), rtol=0, atol=2e-5)
            assert np.array_equal(q2[t, h, 256:], qg[t, h, 256:])   # the gate half is left alone
        for h in range(nkv):
            assert np.allclose(k2[t, h], want(k[t, h], kn, pos0 + t), rtol=0, atol=2e-5)
            assert np.array_equal(kc[pos0 + t, h].view(np.float16), k2[t, h].astype(np.float16))
            assert np.array_equal(vc[pos0 + t, h].view(np.float16), v[t, h].astype(np.float16))
    assert not kc[:pos0].any() and not kc[pos0 + T:].any()
    # the rotary's defining property: q . k after rotation depends on the positions only through their difference
    q1, k1 = prep(oracle, qg[:1], k[:1], v[:1], qn, kn, kc.copy(), vc.copy(), nq, nkv, 7)
    q3, _ = prep(oracle, qg[:1], k[:1], v[:1], qn, kn, kc.copy(), vc.copy(), nq, nkv, 9)
    qa, ka = prep(oracle, qg[:1], k[:1], v[:1], qn, kn, kc.copy(), vc.copy(), nq, nkv, 3)
    qb, _ = prep(oracle, qg[:1], k[:1], v[:1], qn, kn, kc.copy(), vc.copy(), nq, nkv, 5)
    assert abs(float(q3[0, 0, :256] @ k1[0, 0]) - float(qb[0, 0, :256] @ ka[0, 0])) < 1e-3


def test_attn_is_softmax_attention(oracle):
    rng = np.random.default_rng(4)
    nq, nkv, T, pos0 = 4, 2, 3, 37
    qg = rng.standard_normal((T, nq, 512)).astype(np.float32)
    kc = rng.standard_normal((64, nkv, 256)).astype(np.float16)
    vc = rng.standard_normal((64, nkv, 256)).astype(np.float16)
    out = np.zeros((T, nq, 256), dtype=np.float32)
    oracle.lib.fnx_o_attn(ol.ptr(qg), ol.ptr(kc), ol.ptr(vc), ol.ptr(out), nq, nkv, 256, T, pos0)
    for t in range(T):
        for h in range(nq):
            kv = h // (nq // nkv)
            ctx = pos0 + t + 1
            s = kc[:ctx, kv].astype(np.float64) @ qg[t, h, :256].astype(np.float64) / 16.0
            p = np.exp(s - s.max())
            p /= p.sum()
            want = (p @ vc[:ctx, kv].astype(np.float64)) / (1 + np.exp(-qg[t, h, 256:].astype(np.float64)))
            assert np.allclose(out[t, h], want, rtol=1e-5, atol=1e-6)
    # one position: the output is that position's v times the gate
    oracle.lib.fnx_o_attn(ol.ptr(qg), ol.ptr(kc), ol.ptr(vc), ol.ptr(out), nq, nkv, 256, 1, 0)
    assert np.allclose(out[0, 3], vc[0, 1].astype(np.float64) / (1 + np.exp(-qg[0, 3, 256:].astype(np.float64))), rtol=1e-6)


def test_decoder_windows_compose(oracle):
    # the rows of one window give the same results as the same rows fed as two windows (causal mask + cache)
    m = td.TinyDecoder(oracle, seed=5)
    a, b = td.OracleSession(m), td.OracleSession(m)
    toks = [7, 11, 400, 23, 999, 5]
    whole = a.verify(toks, 0)
    first, second = b.verify(toks[:2], 0), b.verify(toks[2:], 2)
    assert np.array_equal(whole["best"], np.concatenate([first["best"], second["best"]]))
    both = np.concatenate([first["hidden"], second["hidden"]])
    assert np.linalg.norm(whole["hidden"] - both) <= 1e-5 * np.linalg.norm(both)
    assert all(np.array_equal(x[0], y[0]) and np.array_equal(x[1], y[1]) for x, y in zip(a.caches, b.caches))
    # the draft layer: rows of the draft head from hidden rows and the next tokens
    d = a.draft(whole["hidden"], toks[1:] + [3], 0)
    assert d["best"].shape == (6,) and np.all(np.isfinite(d["hidden"]))

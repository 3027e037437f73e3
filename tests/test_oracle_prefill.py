"""The prompt path's oracle functions against independent statements of the same mathematics (numpy, f64)."""
import numpy as np

from fnx_gpu import random_iq3s


def test_dequant_f16_is_the_f32_value_rounded_once(oracle):
    rng = np.random.default_rng(5)
    blocks = random_iq3s(rng, 64, dmax=2e-2)
    f32 = oracle.iq3s_dequant(blocks)
    assert np.array_equal(oracle.iq3s_dequant_f16(blocks).view(np.uint16), f32.astype(np.float16).view(np.uint16))
    # tiny d: the products land among f16's subnormals and are still rounded to nearest even
    small = random_iq3s(rng, 8, dmax=3e-6)
    assert np.array_equal(oracle.iq3s_dequant_f16(small).view(np.uint16), oracle.iq3s_dequant(small).astype(np.float16).view(np.uint16))


def test_f32_f16_matches_ieee(oracle):
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.standard_normal(4096) * 10.0 ** rng.integers(-8, 5, 4096), [0.0, -0.0, 65504.0, 65520.0, 1e-8, 6.1e-5]]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_f16(x).view(np.uint16), want)


def test_moe_mma_is_a_matrix_product_of_the_rounded_operands(oracle):
    rng = np.random.default_rng(7)
    nrows, ncols, nexp, pf = 32, 512, 3, 64
    w = random_iq3s(rng, nexp * nrows * ncols // 256, dmax=2e-2)
    stride = nrows * ncols // 256 * 110
    x16 = rng.standard_normal((40, ncols)).astype(np.float16)
    jobs = np.zeros((3, 2 + 2 * pf), dtype=np.int32)
    rows_of = [(2, list(range(0, 17))), (0, [39, 3, 5]), (1, list(range(10, 40)))]
    at = 0
    for j, (e, ys) in enumerate(rows_of):
        jobs[j, 0], jobs[j, 1] = e, len(ys)
        jobs[j, 2:2 + len(ys)] = ys
        jobs[j, 2 + pf:2 + pf + len(ys)] = np.arange(at, at + len(ys))
        at += len(ys)
    got = oracle.moe_mma(w, stride, nrows, ncols, jobs, pf, x16, at)
    at = 0
    for e, ys in rows_of:
        W = oracle.iq3s_dequant(w[e * stride:(e + 1) * stride]).astype(np.float16).astype(np.float64).reshape(nrows, ncols)
        want = x16[ys].astype(np.float64) @ W.T
        assert np.array_equal(got[at:at + len(ys)], want.astype(np.float32))
        at += len(ys)


def test_swiglu_h16(oracle):
    rng = np.random.default_rng(8)
    gu = (rng.standard_normal((9, 128)) * 3).astype(np.float32)
    got = oracle.swiglu_h16(gu, 64).astype(np.float64)
    g, u = gu[:, :64].astype(np.float64), gu[:, 64:].astype(np.float64)
    want = g / (1 + np.exp(-g)) * u
    # f32 arithmetic then one rounding to f16: within one f16 ulp of the exact value
    ulp = np.maximum(np.abs(want), 2.0 ** -14) * 2.0 ** -10
    assert np.all(np.abs(got - want) <= ulp)


def test_prefill_layer_equals_its_parts(oracle):
    rng = np.random.default_rng(9)
    n, ff, nexp, topk, Cn = 256, 256, 8, 2, 70
    nb = lambda rows, cols: rows * cols // 256
    gu = random_iq3s(rng, nexp * nb(2 * ff, n), dmax=2e-2)
    down = random_iq3s(rng, nexp * nb(n, ff), dmax=2e-2)
    sh_gu, sh_down = random_iq3s(rng, nb(2 * ff, n), dmax=2e-2), random_iq3s(rng, nb(n, ff), dmax=2e-2)
    router = (rng.standard_normal((nexp + 1, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((Cn, n)).astype(np.float32)
    r = oracle.moe_prefill_layer(n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x)
    # the same from dense f64 algebra on the rounded operands
    logits = oracle.gemv_f32(router, x)
    assert np.array_equal(r["logits"], logits)
    topi, topw = oracle.topk_logits(logits, nexp, topk)
    assert np.array_equal(r["topi"], topi)
    xh = x.astype(np.float16).astype(np.float64)
    deq = lambda b, rows, cols: oracle.iq3s_dequant(b).astype(np.float16).astype(np.float64).reshape(rows, cols)

    def ffn(Wgu, Wd, rows):
        g = (rows @ Wgu.T).astype(np.float32)
        h = oracle.swiglu_h16(g, ff).astype(np.float64)
        return (h @ Wd.T).astype(np.float32)

    gs, ds = 2 * ff * n // 256 * 110, n * ff // 256 * 110
    want = np.zeros((Cn, n), dtype=np.float64)
    for t in range(Cn):
        for k in range(topk):
            e = topi[t, k]
            want[t] += topw[t, k] * ffn(deq(gu[e * gs:(e + 1) * gs], 2 * ff, n), deq(down[e * ds:(e + 1) * ds], n, ff), xh[t:t + 1])[0]
    sh = ffn(deq(sh_gu, 2 * ff, n), deq(sh_down, n, ff), xh)
    want += (1 / (1 + np.exp(-logits[:, nexp].astype(np.float64))))[:, None] * sh
    assert np.linalg.norm(r["out"] - want) <= 1e-6 * np.linalg.norm(want)
    assert r["njobs"] == sum((np.count_nonzero(topi == e) + 63) // 64 for e in range(nexp))

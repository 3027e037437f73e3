"""fnx_top_tokens / fnx_penalize_row (kernels.hpp:434-447, topk.cuh) through the C ABI against the CPU oracle.
Bar: bit-exact - the candidates' ids and values, the row as changed in place, the error word."""
import numpy as np
import pytest

import fnx_gpu
import oracle_lib as ol
from test_oracle_sampler import o_top_tokens, pack_lists

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return fnx_gpu.Dev()


def d_top_tokens(dev, logits, v0=0, pen=None, par=None, bias=None, lists=True):
    t = dev.torch
    T, n = logits.shape
    L = dev.up(np.ascontiguousarray(logits, dtype=np.float32))
    a = pack_lists(T, pen, par, bias)
    d = {k: dev.up(v) for k, v in a.items() if k != "stride"}
    ov, oi, err = dev.zeros((T, 64), t.float32), dev.zeros((T, 64), t.int32), dev.zeros(1, t.int32)
    p = (lambda k: d[k].data_ptr()) if lists else (lambda k: None)
    dev.ok(dev.lib.fnx_top_tokens(L.data_ptr(), n, T, v0, p("pen_tok"), p("pen_cnt"), p("pen_n"), a["stride"], p("par"), p("bias_tok"), p("bias_val"),
                                  p("bias_off"), p("bias_n"), ov.data_ptr(), oi.data_ptr(), err.data_ptr(), dev.st()))
    dev.sync()
    return ov.cpu().numpy(), oi.cpu().numpy(), L.cpu().numpy(), int(err.item())


def same(got, want):
    assert np.array_equal(got[1], want[1]), "candidate ids"
    assert np.array_equal(got[0].view(np.uint32), want[0].view(np.uint32)), "candidate values"
    assert np.array_equal(got[2].view(np.uint32), want[2].view(np.uint32)), "the rows as changed in place"
    assert got[3] == want[3]


@pytest.mark.parametrize("n,T", [(64, 1), (65, 3), (1000, 16), (2560, 2), (2561, 2), (5121, 5), (151936, 16), (327680, 1)])
def test_top_tokens_shapes(dev, oracle, n, T):
    print(f"case top_tokens n={n} T={T}", flush=True)
    rng = np.random.default_rng(n + T)
    x = rng.standard_normal((T, n)).astype(np.float32)
    same(d_top_tokens(dev, x, v0=11), o_top_tokens(oracle, x, v0=11))
    same(d_top_tokens(dev, x, lists=False), o_top_tokens(oracle, x))


def test_top_tokens_ties_zeros_and_non_finite(dev, oracle):
    rng = np.random.default_rng(8)
    n = 6000
    x = rng.standard_normal((6, n)).astype(np.float32)
    x[0] = 0.75                                          # a whole row of equal logits: ids 0 .. 63
    x[1, rng.integers(0, n, n // 2)] = 2.5               # a tie far wider than the candidates, at the top
    x[2] = np.round(x[2] * 2) / 2                        # ties at the threshold
    x[3, :] = -0.0
    x[3, 3000:3070] = 0.0                                # signed zeros: +0 above -0
    x[4, 17], x[4, 4000] = np.inf, -np.inf
    x[5, 5999] = np.nan
    print("case top_tokens ties / zeros / non-finite", flush=True)
    got, want = d_top_tokens(dev, x), o_top_tokens(oracle, x)
    same(got, want)
    assert got[3] == 16 and list(got[1][0]) == list(range(64)) and list(got[1][3]) == list(range(3000, 3064))
    # the ties' ids come out ascending whatever slice they lie in
    tied = got[1][1][got[0][1] == 2.5]
    assert tied.size > 32 and np.all(np.diff(tied) > 0) and tied[0] < 64


def test_top_tokens_bias_and_penalties(dev, oracle):
    rng = np.random.default_rng(9)
    n, T, v0 = 151936, 16, 0
    x = rng.standard_normal((T, n)).astype(np.float32)
    pen, par, bias = [], [], []
    for t in range(T):
        k = int(rng.integers(0, 4096))
        toks = rng.choice(n, k, replace=False)
        pen.append([(int(a), int(c)) for a, c in zip(toks, rng.integers(0, 5, k))] + [(-3, 1), (n + 5, 2)])
        par.append((float(rng.choice([1.0, 1.1, 1.5])), float(rng.choice([0.0, 0.2])), float(rng.choice([0.0, 0.4]))))
        top = np.argsort(-x[t])[:8]
        bias.append([(int(a), float(b)) for a, b in zip(top, rng.standard_normal(8) * 4)] + [(int(rng.integers(0, n)), 50.0)] if t % 2 else [])
        if t % 3 == 0:   # penalties on the row's best tokens, so that they matter
            pen[-1] += [(int(a), 3) for a in np.argsort(-x[t])[8:40] if a not in set(toks.tolist())]
    print("case top_tokens bias + penalties, 16 x 151,936", flush=True)
    same(d_top_tokens(dev, x, v0=v0, pen=pen, par=par, bias=bias), o_top_tokens(oracle, x, v0=v0, pen=pen, par=par, bias=bias))
    # a vocabulary slice that starts at v0: lists hold global token ids
    xs = x[:, :4000].copy()
    pen2 = [[(500 + int(a), 2) for a in rng.choice(4000, 50, replace=False)] for _ in range(T)]
    same(d_top_tokens(dev, xs, v0=500, pen=pen2, par=par), o_top_tokens(oracle, xs, v0=500, pen=pen2, par=par))


def test_penalize_row(dev, oracle):
    rng = np.random.default_rng(10)
    n, k = 5000, 300
    row = rng.standard_normal(n).astype(np.float32)
    packed = np.concatenate([[k], rng.choice(n + 10, k, replace=False) - 5, rng.integers(0, 4, k)]).astype(np.int32)
    par = np.array([1.25, 0.1, 0.3], np.float32)
    want = row.copy()
    oracle.lib.fnx_o_penalize_row(ol.ptr(want), n, ol.ptr(packed), ol.ptr(par))
    d, dpen, dpar = dev.up(row), dev.up(packed), dev.up(par)   # named: a device buffer lives as long as its tensor does
    dev.ok(dev.lib.fnx_penalize_row(d.data_ptr(), n, dpen.data_ptr(), dpar.data_ptr(), dev.st()))
    dev.sync()
    assert np.array_equal(d.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_top_tokens_bad_arguments(dev):
    t = dev.torch
    b = dev.zeros(4096, t.float32)
    assert dev.lib.fnx_top_tokens(b.data_ptr(), 63, 1, 0, None, None, None, 0, None, None, None, None, None, b.data_ptr(), b.data_ptr(), b.data_ptr(), dev.st()) != 0
    assert b"smaller than the candidates" in dev.lib.fnx_last_error()
    assert dev.lib.fnx_top_tokens(b.data_ptr(), 64, 17, 0, None, None, None, 0, None, None, None, None, None, b.data_ptr(), b.data_ptr(), b.data_ptr(), dev.st()) != 0
    assert dev.lib.fnx_top_tokens(b.data_ptr(), 64, 1, 0, None, None, b.data_ptr(), 0, None, None, None, None, None, b.data_ptr(), b.data_ptr(), b.data_ptr(), dev.st()) != 0

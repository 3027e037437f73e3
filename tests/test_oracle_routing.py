"""Pins of the oracle's routing, job building, SwiGLU, combine, argmax, lookup, acceptance and prefill permutation."""
import numpy as np
import pytest

import oracle_lib as ol


# ---------------------------------------------------------------- f32 mat-vec
def test_gemv_f32_exact_on_small_integers(oracle):
    # small integers: every partial sum is exact in f32, so any summation order gives the same bits
    rng = np.random.default_rng(10)
    W = rng.integers(-8, 9, size=(37, 512)).astype(np.float32)
    x = rng.integers(-8, 9, size=(5, 512)).astype(np.float32)
    got = oracle.gemv_f32(W, x)
    want = (x.astype(np.int64) @ W.astype(np.int64).T).astype(np.float32)
    assert np.array_equal(got, want)


def test_gemv_f32_close_to_f64(oracle):
    rng = np.random.default_rng(11)
    W = (rng.standard_normal((513, 2048)) * 0.02).astype(np.float32)
    x = rng.standard_normal((16, 2048)).astype(np.float32)
    got = oracle.gemv_f32(W, x)
    want = x.astype(np.float64) @ W.astype(np.float64).T
    assert np.abs(got - want).max() < 2e-6 * np.abs(want).max() + 1e-6


def test_gemv_bf16_equals_f32_on_widened_weights(oracle):
    rng = np.random.default_rng(12)
    Wb = rng.integers(0, 65536, size=(9, 256), dtype=np.uint16)
    Wb = np.where(((Wb >> 7) & 0xFF) == 0xFF, 0, Wb).astype(np.uint16)   # no inf / NaN
    Wf = (Wb.astype(np.uint32) << 16).view(np.float32)
    x = rng.standard_normal((3, 256)).astype(np.float32)
    assert np.array_equal(oracle.gemv_bf16(Wb, x).view(np.uint32), oracle.gemv_f32(Wf, x).view(np.uint32))


# ---------------------------------------------------------------- top-k
def brute_topk(row, k):
    order = sorted(range(len(row)), key=lambda i: (-row[i], i))
    return order[:k]


def test_topk_against_sort(oracle):
    rng = np.random.default_rng(13)
    logits = rng.standard_normal((16, 513)).astype(np.float32)
    topi, topw = oracle.topk_logits(logits, 512, 10)
    for t in range(16):
        assert list(topi[t]) == brute_topk(logits[t, :512], 10)
        l = logits[t, topi[t]].astype(np.float64)
        w = np.exp(l - l[0])
        assert np.allclose(topw[t], w / w.sum(), rtol=1e-6)
        assert abs(topw[t].sum() - 1) < 1e-6
        assert np.all(np.diff(topw[t]) <= 0)


def test_topk_ties_take_lower_index(oracle):
    logits = np.zeros((2, 65), dtype=np.float32)
    logits[1, [5, 9, 40]] = 1.0
    logits[1, [3, 50]] = 0.5
    topi, topw = oracle.topk_logits(logits, 64, 10)
    assert list(topi[0]) == list(range(10))
    assert np.allclose(topw[0], 0.1)
    assert list(topi[1]) == [5, 9, 40, 3, 50, 0, 1, 2, 4, 6]


def test_two_routing_definitions_agree(oracle):
    # kernels.cu:338-378 (softmax over all, top-k of probabilities, renormalise) vs moe.cuh:382-411 (top-k by logit,
    # exp(l - l0) / sum): the same picks and, up to rounding, the same weights
    rng = np.random.default_rng(14)
    logits = (rng.standard_normal((64, 512)) * 2).astype(np.float32)
    i1, w1 = oracle.topk_logits(logits, 512, 10)
    i2, w2 = oracle.topk_softmax(logits, 512, 10)
    assert np.array_equal(i1, i2)
    assert np.allclose(w1, w2, rtol=2e-6, atol=1e-9)


def test_topk_ignores_the_shared_gate_column(oracle):
    logits = np.zeros((1, 9), dtype=np.float32)
    logits[0, 8] = 100.0   # the row's last column is the shared expert's gate, not an expert
    topi, _ = oracle.topk_logits(logits, 8, 3)
    assert list(topi[0]) == [0, 1, 2]


def scarce_logits(rng, T, nexp):
    """rows with fewer selectable logits than picks: -inf masks and NaN entries; the last row has none at all"""
    lg = rng.standard_normal((T, nexp + 1)).astype(np.float32)
    lg[0, :nexp] = -np.inf
    lg[0, [7, 3, nexp - 1]] = [0.5, 0.25, 1.5]          # three finite logits
    if T > 1:
        lg[1, :nexp] = np.nan
        lg[1, [1, 4]] = [2.0, 2.0]                       # two finite logits, tied
    if T > 2:
        lg[2, 0:nexp:2] = -np.inf                        # half of the experts masked: enough left, nothing is filled in
    if T > 3:
        lg[T - 1, :nexp] = -np.inf                       # nothing to pick
        lg[T - 1, 5] = np.nan
    return lg


def test_topk_with_fewer_finite_logits_than_picks(oracle):
    rng = np.random.default_rng(16)
    nexp, topk = 64, 6
    lg = scarce_logits(rng, 5, nexp)
    topi, topw = oracle.topk_logits(lg, nexp, topk)
    for t in range(5):
        assert len(set(topi[t].tolist())) == topk and topi[t].min() >= 0 and topi[t].max() < nexp
    assert list(topi[0]) == [nexp - 1, 7, 3, 0, 1, 2]       # the finite ones by value, then the lowest indexes not yet picked
    e = np.exp(np.array([0.0, -1.0, -1.25]))
    assert np.allclose(topw[0, :3], e / e.sum(), rtol=1e-6) and np.all(topw[0, 3:] == 0)
    assert list(topi[1]) == [1, 4, 0, 2, 3, 5]
    assert np.allclose(topw[1, :2], 0.5) and np.all(topw[1, 2:] == 0)
    assert list(topi[2]) == brute_topk(np.where(np.isinf(lg[2, :nexp]), -1e30, lg[2, :nexp]), topk)
    assert abs(topw[2].sum() - 1) < 1e-6
    assert list(topi[4]) == list(range(topk)) and np.all(topw[4] == 0)
    # every job holds a token at most once
    gu, dn = oracle.jobs(topi)
    assert all(int(j["n"]) <= 5 for j in gu)
    assert sum(int(j["n"]) for j in gu) == 5 * topk


# ---------------------------------------------------------------- jobs
def test_jobs_invariants(oracle):
    rng = np.random.default_rng(15)
    T, K = 16, 10
    topi = np.stack([rng.choice(40, K, replace=False) for _ in range(T)]).astype(np.int32)
    gu, dn = oracle.jobs(topi)
    flat = topi.reshape(-1)
    first_seen = list(dict.fromkeys(flat.tolist()))
    assert [int(j["w"]) for j in gu] == first_seen and [int(j["w"]) for j in dn] == first_seen
    assert sum(int(j["n"]) for j in gu) == T * K
    seen = set()
    for jg, jd in zip(gu, dn):
        n = int(jg["n"])
        assert n == int(jd["n"]) and 1 <= n <= T
        pairs = jg["out"][:n]
        assert np.all(np.diff(pairs) > 0), "pairs of a job in ascending order"
        assert np.array_equal(jg["y"][:n], pairs // K)
        assert np.array_equal(jd["y"][:n], pairs) and np.array_equal(jd["out"][:n], pairs)
        assert np.all(flat[pairs] == jg["w"])
        assert seen.isdisjoint(pairs.tolist())
        seen.update(pairs.tolist())
    assert seen == set(range(T * K))


# ---------------------------------------------------------------- swiglu, combine
def test_swiglu_q8_1_against_f64(oracle):
    rng = np.random.default_rng(16)
    gu = rng.standard_normal((6, 2 * 128)).astype(np.float32) * 3
    hq = oracle.swiglu_stacked_q8_1(gu, 128)
    g, u = gu[:, :128].astype(np.float64), gu[:, 128:].astype(np.float64)
    h = g / (1 + np.exp(-g)) * u
    b = hq.reshape(6, 4, 36)
    d = b[:, :, 0:2].copy().view(np.float16).astype(np.float64)[..., 0]
    back = (b[:, :, 4:].view(np.int8).astype(np.float64) * d[..., None]).reshape(6, 128)
    dmax = np.repeat(d, 32, axis=1)
    assert np.all(np.abs(back - h) <= 0.51 * dmax + 1e-3 * np.abs(h))
    # the two entry forms agree
    assert np.array_equal(hq, oracle.swiglu_q8_1(gu[:, :128].copy(), gu[:, 128:].copy()))


def test_combine_against_f64(oracle):
    rng = np.random.default_rng(17)
    T, K, n = 4, 10, 64
    part = rng.standard_normal((T * K, n)).astype(np.float32)
    topw = rng.random((T, K)).astype(np.float32)
    sh = rng.standard_normal((T, n)).astype(np.float32)
    shl = rng.standard_normal(T).astype(np.float32)
    got = oracle.moe_combine(part, topw, sh, shl)
    want = np.einsum("tk,tkn->tn", topw.astype(np.float64), part.reshape(T, K, n).astype(np.float64))
    want += (1 / (1 + np.exp(-shl.astype(np.float64))))[:, None] * sh
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # one expert with weight 1, gate logit very negative: the output is that expert's row
    topw[:] = 0
    topw[:, 3] = 1
    got = oracle.moe_combine(part, topw, sh, np.full(T, -100, dtype=np.float32))
    assert np.array_equal(got, part.reshape(T, K, n)[:, 3])


# ---------------------------------------------------------------- argmax
def test_argmax_brute_force_ties_and_signs(oracle):
    rng = np.random.default_rng(18)
    logits = rng.standard_normal((4, 1000)).astype(np.float32)
    logits[1] = -np.abs(logits[1]) - 1      # all negative
    logits[2, [17, 400, 999]] = 9.0         # a three-way tie: the lowest index wins
    logits[3] = 0.0
    logits[3, 5] = -0.0                     # +0 sorts above -0 in key order; index 0 holds +0
    bv, bi, err = oracle.argmax(logits, v0=100)
    assert err == 0
    assert bi[0] == 100 + int(np.argmax(logits[0])) and bv[0] == logits[0].max()
    assert bi[1] == 100 + int(np.argmax(logits[1])) and bv[1] == logits[1].max()
    assert bi[2] == 117 and bv[2] == 9.0
    assert bi[3] == 100


def test_argmax_flags_non_finite(oracle):
    logits = np.zeros((2, 1000), dtype=np.float32)
    logits[1, 7] = np.nan
    _, _, err = oracle.argmax(logits)
    assert err & 16
    logits[1, 7] = np.inf
    _, _, err = oracle.argmax(logits)
    assert err & 16
    logits[1, 7] = 3.0e38
    bv, bi, err = oracle.argmax(logits)
    assert err == 0 and bi[1] == 7


# ---------------------------------------------------------------- prompt lookup
def brute_lookup(ctx, lk, d1, key_n=3, lookup_min=3):
    """session.hpp:55-57 restated from the prose: latest earlier place of the last key_n tokens; drafts only if its
    continuation starts with d1; as many as the match is long, lookup_min..lk; clipped at the end of the context."""
    n = len(ctx)
    if lk == 0 or n <= key_n:
        return [], -1
    key = ctx[n - key_n:]
    places = [s for s in range(n - key_n) if ctx[s:s + key_n] == key]
    if not places:
        return [], -1
    s = places[-1]
    if not (s + key_n < n and (d1 < 0 or ctx[s + key_n] == d1)):
        return [], -1
    m = key_n
    while m < lk and s - 1 - (m - key_n) >= 0 and ctx[s - 1 - (m - key_n)] == ctx[n - key_n - 1 - (m - key_n)]:
        m += 1
    k = min(lk, max(lookup_min, m))
    out = ctx[s + key_n:min(n, s + key_n + k)]
    for i, t in enumerate(out):
        if t >= 1 << 30:
            out = out[:i]
            break
    return out, s


@pytest.mark.parametrize("key_n", [2, 3, 4])
def test_lookup_against_brute_force(oracle, key_n):
    rng = np.random.default_rng(19 + key_n)
    for case in range(300):
        n = int(rng.integers(1, 60))
        ctx = rng.integers(0, 4, size=n).tolist()   # a tiny alphabet: many repeats
        lk = int(rng.integers(0, 16))
        d1 = int(rng.integers(-1, 4))
        got, match = oracle.lookup_drafts(ctx, lk, d1, key_n)
        want, wmatch = brute_lookup(ctx, lk, d1, key_n)
        assert list(got) == want and match == wmatch, (ctx, lk, d1)
        if len(got):
            assert d1 < 0 or got[0] == d1


def test_lookup_edge_cases(oracle):
    assert len(oracle.lookup_drafts([1, 2, 3], 15, -1)[0]) == 0            # ctx.size() <= 3
    assert len(oracle.lookup_drafts([1, 2, 3, 1, 2, 3], 0, -1)[0]) == 0    # lk = 0
    # a match whose continuation runs to the end of the context is clipped there
    got, match = oracle.lookup_drafts([7, 1, 2, 3, 9, 1, 2, 3], 15, 9)
    assert list(got) == [9, 1, 2] and match == 1                           # a 3-token match offers LOOKUP_MIN drafts
    got, match = oracle.lookup_drafts([5, 5, 5, 5], 15, 5)
    assert list(got) == [5] and match == 0                                 # 3 wanted, one left before the end
    got, match = oracle.lookup_drafts([8, 5, 5, 5, 5, 5], 15, -1)
    assert list(got) == [5] and match == 2                                 # the latest place overlaps the key itself
    # only the latest match is examined: its continuation is not d1, so no drafts even though an older one fits
    got, match = oracle.lookup_drafts([1, 2, 3, 5, 0, 1, 2, 3, 6, 0, 1, 2, 3], 15, 5)
    assert len(got) == 0 and match == -1
    # an image cell ends the drafts
    got, _ = oracle.lookup_drafts([1, 2, 3, 4, (1 << 30) + 5, 6, 1, 2, 3], 15, 4)
    assert list(got) == [4]


def test_lookup_two_reference_forms_agree_on_long_matches(oracle):
    # tools/fnx_run.cpp:1046-1059 offers a fixed lk drafts; session.cpp's offers as many as the match is long. They
    # agree whenever the match is at least lk long.
    rng = np.random.default_rng(23)
    base = rng.integers(0, 1000, size=400).tolist()
    for lk in (3, 5, 15):
        span = base[100:100 + lk + 8]
        ctx = base + span[:lk + 4]          # the last lk+4 tokens copy an earlier run
        d1 = span[lk + 4]
        a, _ = oracle.lookup_drafts(ctx, lk, d1)
        b = oracle.lookup_fixed(ctx, lk, d1)
        assert len(a) == lk and list(a) == list(b)


# ---------------------------------------------------------------- acceptance
def test_accept_speculative_equals_greedy(oracle):
    # fnx_run spec's invariant (tools/fnx_run.cpp:1198-1238): whatever the drafts, the accepted tokens are the ones
    # plain greedy decoding produces. Model: next(token history) is a fixed function of the last token.
    rng = np.random.default_rng(24)
    nxt = rng.integers(0, 50, size=50)
    for bad in (0.0, 0.3, 1.0):
        seq = [3]
        while len(seq) < 200:
            R = int(rng.integers(1, 17))
            rows = [seq[-1]]
            for _ in range(R - 1):      # drafts: right with probability 1 - bad
                rows.append(int(nxt[rows[-1]]) if rng.random() >= bad else int(rng.integers(0, 50)))
            o = [int(nxt[r]) for r in rows]     # the verify window's greedy picks, row by row
            n = oracle.accept_greedy(rows, o)
            assert 1 <= n <= R
            seq.extend(o[:n])
        greedy = [3]
        while len(greedy) < len(seq):
            greedy.append(int(nxt[greedy[-1]]))
        assert seq == greedy


# ---------------------------------------------------------------- prefill permutation
def test_pf_jobs_brute_force(oracle):
    rng = np.random.default_rng(25)
    C, K, E, PJ = 96, 10, 32, 64
    p = 1.0 / np.arange(1, E + 1) ** 1.1
    p /= p.sum()
    topi = np.stack([rng.choice(E, K, replace=False, p=p) for _ in range(C)]).astype(np.int32)
    gu, dn, cnt = oracle.pf_jobs(topi, E, PJ)
    flat = topi.reshape(-1)
    assert np.array_equal(cnt, np.bincount(flat, minlength=E))
    assert len(gu) == sum((c + PJ - 1) // PJ for c in cnt)
    assert sum(int(j[1]) for j in gu) == C * K
    at = 0
    for e in range(E):
        pairs = np.nonzero(flat == e)[0]
        for s in range(0, len(pairs), PJ):
            chunk = pairs[s:s + PJ]
            j, d = gu[at], dn[at]
            assert j[0] == e and j[1] == len(chunk) and d[0] == e and d[1] == len(chunk)
            assert np.array_equal(j[2 + PJ:2 + PJ + len(chunk)], chunk)
            assert np.array_equal(j[2:2 + len(chunk)], chunk // K)
            assert np.array_equal(d[2:2 + len(chunk)], chunk) and np.array_equal(d[2 + PJ:2 + PJ + len(chunk)], chunk)
            at += 1
    assert at == len(gu)


def test_the_fixed_exp_is_exp(oracle):
    """include/fnx_expf.h (the exp behind sigm, silu_ and the routing weights on both sides) against numpy's float64 exp:
    within 1.1 units in the last place over its whole range, exact at 0, monotone over a dense sweep, 0 / inf / NaN where its
    header says. A dropped term of the polynomial, a wrong split of ln 2 or a wrong scaling by 2^n fails the first bar."""
    x = np.concatenate([np.linspace(-87.3, 88.72, 400001), np.random.default_rng(5).uniform(-20, 20, 200000),
                        np.array([0.0, -0.0, 1.0, -1.0, 1e-8, -1e-8, 87.0, -87.0, 88.72, -87.3])]).astype(np.float32)
    got = oracle.expf(x).astype(np.float64)
    want = np.exp(x.astype(np.float64))
    ulp = np.spacing(want.astype(np.float32)).astype(np.float64)
    assert np.all(np.isfinite(got))
    assert np.max(np.abs(got - want) / ulp) <= 1.1, "within 1.1 units in the last place (measured: 1.03)"
    assert oracle.expf(np.array([0.0], dtype=np.float32))[0] == 1.0
    s = np.sort(x)
    assert np.all(np.diff(oracle.expf(s)) >= 0), "monotone"
    edge = oracle.expf(np.array([-87.31, -1000.0, -np.inf, 88.73, 1000.0, np.inf, np.nan], dtype=np.float32))
    assert list(edge[:3]) == [0.0, 0.0, 0.0] and np.all(np.isinf(edge[3:6])) and np.isnan(edge[6])

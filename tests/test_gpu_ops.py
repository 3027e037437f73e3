"""Parity of the HIP operators with the CPU oracle, through the C ABI, on the same seeded inputs.

Bar: bit-exact for bytes, integers and indices (q8_1 blocks, router logits, routing picks, jobs, argmax, drafts,
accepted lengths); relative L2 <= 1e-3 for float outputs of the IQ3_S products (measured: ~1e-7).
"""
import numpy as np
import pytest

import fnx_gpu
from fnx_gpu import JOB_DTYPE, random_iq3s

pytestmark = pytest.mark.gpu

REL_L2 = 1e-3


def rel_l2(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return fnx_gpu.Dev()


# ---------------------------------------------------------------- q8_1
@pytest.mark.parametrize("rows,n", [(1, 2048), (16, 2048), (5, 512), (3, 32)])
def test_quantize_q8_1_bit_exact(dev, oracle, rows, n):
    print(f"case quantize rows={rows} n={n}", flush=True)
    rng = np.random.default_rng(100 + rows)
    x = rng.standard_normal((rows, n)).astype(np.float32)
    x[0, :32] = 0.0
    if n >= 64:
        x[0, 32:64] = np.arange(32) * 0.5 - 7.75   # exact halves: rounds away from zero
    assert np.array_equal(dev.quantize_q8_1(x), oracle.quantize_q8_1(x))


# ---------------------------------------------------------------- router mat-vec
@pytest.mark.parametrize("rows,n,T", [(513, 2048, 16), (513, 2048, 1), (37, 256, 5), (8, 4096, 3), (513, 2048, 100), (30, 512, 17), (3, 256, 64)])
def test_gemv_f32_bit_exact(dev, oracle, rows, n, T):
    print(f"case gemv_f32 rows={rows} n={n} T={T}", flush=True)
    rng = np.random.default_rng(200 + rows + T)
    W = (rng.standard_normal((rows, n)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, n)).astype(np.float32)
    assert np.array_equal(dev.gemv(W, x).view(np.uint32), oracle.gemv_f32(W, x).view(np.uint32))


# 64 rows of x and more against f32 weights with rows of a multiple of 2048: the tiles on the matrix cores (ragged last
# tiles of both kinds, weight rows past the last full 32, more than one patch of tiles, rows of 4096), with values over
# many binades so that a sum's bits depend on the order of its adds
@pytest.mark.parametrize("rows,n,T", [(513, 2048, 512), (96, 2048, 70), (290, 2048, 200), (64, 4096, 64), (35, 2048, 129), (33, 4096, 66), (65, 3072, 96)])
def test_gemv_f32_many_rows_bit_exact(dev, oracle, rows, n, T):
    print(f"case gemv_f32 (tiles) rows={rows} n={n} T={T}", flush=True)
    rng = np.random.default_rng(230 + rows + T)
    W = (rng.standard_normal((rows, n)) * np.exp2(rng.integers(-12, 4, (rows, n)))).astype(np.float32)
    x = (rng.standard_normal((T, n)) * np.exp2(rng.integers(-8, 8, (T, n)))).astype(np.float32)
    x[rng.integers(0, T, 40), rng.integers(0, n, 40)] = 0.0
    assert np.array_equal(dev.gemv(W, x).view(np.uint32), oracle.gemv_f32(W, x).view(np.uint32))


def test_gemv_f32_sum_does_not_depend_on_T(dev):
    """A size-independent property at a size the oracle takes long for: a sum's bits do not depend on how many rows of x a
    call brings, so 4,099 rows in one call (the matrix cores' tiles, several patches of them, a ragged last tile, the 513th
    weight row with the loading waves) must equal the same rows in calls of 16 and fewer (the vector units' kernel)."""
    rows, n, T = 513, 2048, 4099
    print(f"case gemv_f32 T-independence rows={rows} n={n} T={T}", flush=True)
    rng = np.random.default_rng(240)
    W = (rng.standard_normal((rows, n)) * np.exp2(rng.integers(-10, 2, (rows, n)))).astype(np.float32)
    x = (rng.standard_normal((T, n)) * np.exp2(rng.integers(-6, 6, (T, n)))).astype(np.float32)
    big = dev.gemv(W, x).view(np.uint32)
    for t0 in list(range(0, 256, 16)) + [1024, 2048, 4080, 4096]:
        small = dev.gemv(W, x[t0:t0 + 16]).view(np.uint32)
        assert np.array_equal(big[t0:t0 + len(small)], small), f"rows {t0}.."


def test_gemv_f32_many_rows_non_finite(dev, oracle):
    """Infinities and NaNs in x and W go through the matrix cores' chains as through fmaf: the same sums are NaN, the same
    +-inf, the finite ones keep their bits (a NaN's payload is not compared)."""
    rows, n, T = 65, 2048, 64
    rng = np.random.default_rng(241)
    W = (rng.standard_normal((rows, n)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, n)).astype(np.float32)
    x[3, 100] = np.inf
    x[5, 7] = -np.inf
    x[9, 2000] = np.nan
    W[10, 100] = 0.0        # inf * 0 = NaN in row 3 x weight row 10
    W[20, 50] = np.inf
    W[64, 1] = np.nan       # the weight row past the tiles
    got, want = dev.gemv(W, x), oracle.gemv_f32(W, x)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    assert np.isnan(want).any() and np.isinf(want).any()


@pytest.mark.parametrize("T", [16, 45])   # 45 rows: the many-rows kernel, with a ragged last group
def test_gemv_bf16_bit_exact(dev, oracle, T):
    rng = np.random.default_rng(210)
    W = ((rng.standard_normal((513, 2048)) * 0.02).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    x = rng.standard_normal((T, 2048)).astype(np.float32)
    assert np.array_equal(dev.gemv(W, x, bf16=True).view(np.uint32), oracle.gemv_bf16(W, x).view(np.uint32))


# ---------------------------------------------------------------- routing
def check_jobs(got, want):
    assert len(got) == len(want)
    for g, w in zip(got, want):
        n = int(w["n"])
        assert int(g["w"]) == int(w["w"]) and int(g["n"]) == n
        assert np.array_equal(g["y"][:n], w["y"][:n]) and np.array_equal(g["out"][:n], w["out"][:n])


@pytest.mark.parametrize("T,nexp,topk", [(16, 512, 10), (1, 512, 10), (7, 64, 4), (16, 1000, 8)])
def test_route_bit_exact(dev, oracle, T, nexp, topk):
    print(f"case route T={T} nexp={nexp} topk={topk}", flush=True)
    rng = np.random.default_rng(300 + T + nexp)
    logits = rng.standard_normal((T, nexp + 1)).astype(np.float32)
    logits[0, :20] = 0.25            # a run of ties: lower indices first
    r = dev.route(logits, nexp, topk)
    topi, topw = oracle.topk_logits(logits, nexp, topk)
    assert np.array_equal(r["topi"], topi)
    assert np.array_equal(r["topw"].view(np.uint32), topw.view(np.uint32))
    gu, dn = oracle.jobs(topi)
    check_jobs(r["gu"], gu)
    check_jobs(r["dn"], dn)
    assert r["njobs"][0] == len(gu) and r["njobs"][1] == len(gu)


@pytest.mark.parametrize("T,nexp,topk", [(16, 512, 10), (5, 64, 6), (16, 1000, 16)])
def test_route_with_fewer_finite_logits_than_picks(dev, oracle, T, nexp, topk):
    # masked (-inf) and NaN logits: the picks stay distinct (the lowest indexes not yet picked, at weight 0) and no job
    # takes a token twice
    from test_oracle_routing import scarce_logits
    print(f"case route scarce T={T} nexp={nexp} topk={topk}", flush=True)
    logits = scarce_logits(np.random.default_rng(305 + T), T, nexp)
    r = dev.route(logits, nexp, topk)
    topi, topw = oracle.topk_logits(logits, nexp, topk)
    assert np.array_equal(r["topi"], topi)
    for t in range(T):
        assert len(set(r["topi"][t].tolist())) == topk
    assert np.array_equal(np.isfinite(r["topw"]), np.ones_like(topw, dtype=bool))
    assert np.array_equal(r["topw"].view(np.uint32), topw.view(np.uint32))
    gu, dn = oracle.jobs(topi)
    check_jobs(r["gu"], gu)
    check_jobs(r["dn"], dn)
    assert max(int(j["n"]) for j in r["gu"][:r["njobs"][0]]) <= T


def test_router_route_fused_bit_exact(dev, oracle):
    rng = np.random.default_rng(310)
    T, n, nexp, topk = 16, 2048, 512, 10
    W = (rng.standard_normal((nexp + 1, n)) * 0.02).astype(np.float32)
    x = rng.standard_normal((T, n)).astype(np.float32)
    r = dev.route(None, nexp, topk, fused_W=W, x=x)
    logits = oracle.gemv_f32(W, x)
    assert np.array_equal(r["logits"].view(np.uint32), logits.view(np.uint32))
    topi, topw = oracle.topk_logits(logits, nexp, topk)
    assert np.array_equal(r["topi"], topi)
    assert np.array_equal(r["topw"].view(np.uint32), topw.view(np.uint32))
    gu, dn = oracle.jobs(topi)
    check_jobs(r["gu"], gu)
    check_jobs(r["dn"], dn)
    assert r["njobs"][0] == len(gu) and r["njobs"][1] == 0   # the second word stays zero (kernels.hpp:279)


# ---------------------------------------------------------------- IQ3_S x q8_1
def test_repack_unit64_bytes(dev):
    # the device's load-time re-laying against a numpy restatement of the layout, out of place and in place
    rng = np.random.default_rng(390)
    raw = random_iq3s(rng, 8 * 37)
    want = fnx_gpu.pack_unit64(raw)
    assert np.array_equal(dev.repack(raw, in_place=False), want)
    assert np.array_equal(dev.repack(raw, in_place=True), want)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("nrows,ncols,T", [(4096, 2048, 1), (4096, 2048, 16), (2048, 512, 16), (1024, 2048, 3), (32, 512, 2),
                                           (16, 256, 5), (64, 1024, 7), (12, 4096, 2), (9, 768, 3), (30, 512, 2), (17, 256, 5)])
def test_gemv_iq3s(dev, oracle, nrows, ncols, T, packed):
    print(f"case gemv_iq3s nrows={nrows} ncols={ncols} T={T} packed={packed}", flush=True)
    if packed and (ncols not in (256, 512, 1024, 2048) or (nrows * ncols) % 2048):
        pytest.skip("the unit64 layout takes whole units only (the raw layout covers this shape)")
    rng = np.random.default_rng(400 + nrows + ncols + T)
    w = random_iq3s(rng, nrows * ncols // 256)
    x = rng.standard_normal((T, ncols)).astype(np.float32)
    got = dev.gemv_iq3s(w, nrows, ncols, x, packed=packed)
    want = oracle.gemv_iq3s(w, nrows, ncols, x)
    assert rel_l2(got, want) <= REL_L2
    assert rel_l2(got, want) <= 1e-5, "in practice only the order of a few float adds differs"


@pytest.mark.parametrize("packed", [False, True])
def test_gemv_iq3s_encoded_gaussian_weights(dev, oracle, packed):
    # benchmark config 1 in small: N(0, 0.02) weights through the encoder, N(0, 1) activations, against the q8_1 oracle
    # and within the int8 path's band of the exact f64 product
    rng = np.random.default_rng(410)
    nrows, ncols = 256, 2048
    w = oracle.iq3s_quantize((rng.standard_normal(nrows * ncols) * 0.02).astype(np.float32))
    for T in (1, 16):
        x = rng.standard_normal((T, ncols)).astype(np.float32)
        got = dev.gemv_iq3s(w, nrows, ncols, x, packed=packed)
        assert rel_l2(got, oracle.gemv_iq3s(w, nrows, ncols, x)) <= 1e-5
        assert rel_l2(got, oracle.gemv_exact(w, nrows, ncols, x)) < 3e-2


# the prompt path's layout under the mat-vec operators: jobs decoded straight into the matrix cores' operands
@pytest.mark.parametrize("nrows,ncols,T", [(4096, 2048, 16), (4096, 2048, 1), (2048, 512, 16), (1024, 2048, 3), (32, 512, 2), (64, 1024, 7),
                                           (48, 1536, 16), (16, 512, 35)])
def test_gemv_iq3s_tile16(dev, oracle, nrows, ncols, T):
    print(f"case gemv_iq3s tile16 nrows={nrows} ncols={ncols} T={T}", flush=True)
    rng = np.random.default_rng(430 + nrows + ncols + T)
    w = random_iq3s(rng, nrows * ncols // 256)
    x = rng.standard_normal((T, ncols)).astype(np.float32)
    got = dev.gemv_iq3s(w, nrows, ncols, x, tile16=True)
    want = oracle.gemv_iq3s(w, nrows, ncols, x)
    assert rel_l2(got, want) <= 1e-5, "only the order of a row's float adds differs"


def test_gemv_iq3s_tile16_encoded_gaussian_weights(dev, oracle):
    rng = np.random.default_rng(431)
    nrows, ncols = 256, 2048
    w = oracle.iq3s_quantize((rng.standard_normal(nrows * ncols) * 0.02).astype(np.float32))
    for T in (1, 16):
        x = rng.standard_normal((T, ncols)).astype(np.float32)
        got = dev.gemv_iq3s(w, nrows, ncols, x, tile16=True)
        assert rel_l2(got, oracle.gemv_iq3s(w, nrows, ncols, x)) <= 1e-5
        assert rel_l2(got, oracle.gemv_exact(w, nrows, ncols, x)) < 3e-2


@pytest.mark.parametrize("packed,tile16", [(False, False), (True, False), (False, True)])
def test_mmvq_jobs_pick_experts_and_rows(dev, oracle, packed, tile16):
    # several experts, jobs with scattered activation and output rows, count read from device memory
    rng = np.random.default_rng(420)
    nexp, nrows, ncols, nrows_y = 6, 96, 2048, 9
    stride = nrows * (ncols // 256) * 110
    w = random_iq3s(rng, nexp * nrows * ncols // 256)
    x = rng.standard_normal((nrows_y, ncols)).astype(np.float32)
    yq = oracle.quantize_q8_1(x)
    jobs = np.zeros(4, dtype=JOB_DTYPE)
    spec = [(5, [0, 3, 8]), (0, [1]), (2, [2, 4, 5, 6, 7]), (3, list(range(9)))]
    at = 0
    for j, (e, ys) in enumerate(spec):
        jobs["w"][j], jobs["n"][j] = e, len(ys)
        jobs["y"][j, :len(ys)] = ys
        jobs["out"][j, :len(ys)] = np.arange(at, at + len(ys))
        at += len(ys)
    got = dev.mmvq(w, stride, nrows, ncols, jobs, yq, at, packed=packed, tile16=tile16)
    want = oracle.mmvq(w, stride, nrows, ncols, jobs, yq, at)
    assert rel_l2(got, want) <= 1e-5
    # with the device count null the host count is used
    assert np.array_equal(dev.mmvq(w, stride, nrows, ncols, jobs, yq, at, njobs_dev=False, packed=packed, tile16=tile16), got)


# ---------------------------------------------------------------- head, drafting, acceptance
def test_argmax_full_vocabulary(dev, oracle):
    rng = np.random.default_rng(500)
    logits = rng.standard_normal((16, 151936)).astype(np.float32)
    logits[3, [100, 70000, 151935]] = 9.5         # a tie: the lowest index
    logits[4] = -np.abs(logits[4]) - 1.0          # all negative
    logits[5, 151935] = 20.0                      # the last column
    bv, bi, err = dev.argmax(logits, v0=7)
    wv, wi, werr = oracle.argmax(logits, v0=7)
    assert np.array_equal(bi, wi) and np.array_equal(bv.view(np.uint32), wv.view(np.uint32)) and err == werr == 0
    assert bi[3] == 107 and bi[5] == 151942


def test_argmax_flags_non_finite(dev, oracle):
    logits = np.zeros((2, 5000), dtype=np.float32)
    logits[1, 4321] = np.nan
    _, _, err = dev.argmax(logits)
    assert err & 16
    logits[1, 4321] = -np.inf
    _, _, err = dev.argmax(logits)
    assert err & 16


def make_context(rng, n=38862, vocab=151936, spans=200):
    ctx = rng.integers(0, vocab, size=n).astype(np.int32)
    for _ in range(spans):
        ln = int(rng.integers(8, 65))
        src = int(rng.integers(0, n - ln))
        dst = int(rng.integers(0, n - ln))
        ctx[dst:dst + ln] = ctx[src:src + ln].copy()
    return ctx


@pytest.mark.parametrize("key_n", [2, 3, 4])
def test_lookup_device_matches_oracle(dev, oracle, key_n):
    rng = np.random.default_rng(600 + key_n)
    ctx = make_context(rng)
    hits = 0
    for case in range(24):
        # end the context inside a copy of an earlier span so the key has an earlier place
        ln = int(rng.integers(8, 65))
        src = int(rng.integers(100, 30000))
        c = np.concatenate([ctx[:38862 - ln], ctx[src:src + ln]]) if case % 4 else ctx[:38862 - case].copy()
        nxt = int(ctx[src + ln]) if case % 4 else -1
        d1 = nxt if case % 3 else -1
        got, match = dev.lookup(c, 15, d1, key_n)
        want, wmatch = oracle.lookup_drafts(c, 15, d1, key_n)
        assert list(got) == list(want) and match == wmatch
        hits += len(want) > 0
    assert hits >= 10
    # edge cases: nothing to match, lk = 0, a short context, an image cell
    for c, lk, d1 in [([1, 2, 3], 15, -1), ([1, 2, 3, 1, 2, 3], 0, -1), ([5, 5, 5, 5], 15, 5), ([8, 5, 5, 5, 5, 5], 15, -1), ([], 15, -1),
                      ([1, 2, 3, 4, (1 << 30) + 5, 6, 1, 2, 3], 15, 4), ([1, 2, 3, 5, 0, 1, 2, 3, 6, 0, 1, 2, 3], 15, 5)]:
        got, match = dev.lookup(c, lk, d1, 3)
        want, wmatch = oracle.lookup_drafts(c, lk, d1, 3)
        assert list(got) == list(want) and match == wmatch, c


def test_accept_device_matches_oracle(dev, oracle):
    rng = np.random.default_rng(700)
    for _ in range(64):
        R = int(rng.integers(1, 17))
        o = rng.integers(0, 1000, size=R).astype(np.int32)
        rows = np.concatenate([[int(rng.integers(0, 1000))], o[:-1]]).astype(np.int32)
        wrong = rng.random(R) > 0.7
        rows[1:][wrong[1:]] += 1
        assert dev.accept(rows, o) == oracle.accept_greedy(rows, o)
    assert dev.accept([4], [9]) == 1
    assert dev.accept([4, 9, 9, 9], [9, 9, 9, 1]) == 4


def test_config3_drafting_and_acceptance(dev, oracle):
    # benchmark config 3: context of 38,862 ids with 200 copied spans, key 3, up to 15 drafts; verify logits 16 x 151,936
    # with the argmax forced to the draft on 70 % of the rows; outputs are the accepted lengths
    rng = np.random.default_rng(800)
    ctx = make_context(rng)
    src = 12345
    c = np.concatenate([ctx[:-40], ctx[src:src + 40]])
    d1 = int(ctx[src + 40])
    drafts, _ = dev.lookup(c, 15, d1, 3)
    wd, _ = oracle.lookup_drafts(c, 15, d1, 3)
    assert list(drafts) == list(wd) and len(drafts) == 15
    rows = np.concatenate([[int(c[-1])], drafts]).astype(np.int32)
    logits = rng.standard_normal((16, 151936)).astype(np.float32)
    keep = rng.random(16) < 0.7
    for t in range(15):
        if keep[t]:
            logits[t, rows[t + 1]] = logits[t].max() + 1.0
    bv, bi, err = dev.argmax(logits)
    wv, wi, _ = oracle.argmax(logits)
    assert np.array_equal(bi, wi) and err == 0
    assert dev.accept(rows, bi) == oracle.accept_greedy(rows, wi)

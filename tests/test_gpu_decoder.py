"""Parity of the norm / dense / attention operators, the reduced decoder's verify window, the draft layer and whole
speculative rounds (benchmark config 4 at test sizes) with the CPU oracle, through the C ABI.

Bar: bit-exact for the dense Q8_0 mat-vec (the summation order is shared with the oracle), for argmax picks, drafts,
accepted lengths and emitted tokens; relative L2 <= 1e-3 for every operator's float output on identical inputs (norms
and attention sum in another order and use the device's rsqrt / exp / sincos; measured 1e-7 .. 1e-6).

Chains of operators (the verify window, the draft layer) re-quantise activations to q8_1 between operators: a last-bit
difference upstream now and then moves one int8 code by one step (1/127 of its block's range), which shows as ~2e-3 in
that row's logits while every other row agrees to 1e-7; cache cells written from such rows (f16) carry the step on to
later rows and windows through the attention. For chains the tests therefore ask: picks identical, every row within
1e-2, and on a fresh cache at least one row within 1e-5 (the arithmetic is the same; the rest is such steps)."""
import ctypes as C

import numpy as np
import pytest

import fnx_gpu
import oracle_lib as ol
import tiny_decoder as td

pytestmark = pytest.mark.gpu
REL_L2 = 1e-3
ROPE = (1e7, 0, 0.0, 0.0, 1.0, 1.0)
YARN = (1e4, 1, 4.0, 20.0, 0.25, float(1.0 + 0.1 * np.log(4.0)))


def rel_l2(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return fnx_gpu.Dev()


def test_rms_norm_rows(dev, oracle):
    rng = np.random.default_rng(801)
    x, w = rng.standard_normal((16, 2048)).astype(np.float32) * 3, rng.standard_normal(2048).astype(np.float32)
    want = np.zeros_like(x)
    oracle.lib.fnx_o_rms_norm_rows(ol.ptr(x), ol.ptr(w), ol.ptr(want), 16, 2048, 1e-6)
    err = float(np.abs(dev.rms_norm_rows(x, w, 1e-6) - want).max())
    assert err <= 3e-6 * float(np.abs(want).max()), err


@pytest.mark.parametrize("n,with_add", [(2048, True), (2048, False), (4096, True), (96, True)])
def test_add_norm_q8_equals_the_three_operators(dev, n, with_add):
    rng = np.random.default_rng(805 + n)
    x, w = rng.standard_normal((5, n)).astype(np.float32) * 2, rng.standard_normal(n).astype(np.float32)
    add = rng.standard_normal((5, n)).astype(np.float32) if with_add else None
    x2, xn, xq = dev.add_norm_q8(x, add, w, 1e-6)
    want_x = x + add if with_add else x
    assert np.array_equal(x2, want_x)
    want_n = dev.rms_norm_rows(want_x, w, 1e-6)
    assert np.array_equal(xn.view(np.uint32), want_n.view(np.uint32))
    assert np.array_equal(xq, dev.quantize_q8_1(want_n))


@pytest.mark.parametrize("T,n,topk", [(16, 2048, 10), (3, 2048, 10), (5, 96, 2)])
def test_combine_add_norm_q8_equals_combine_then_add_norm(dev, oracle, T, n, topk):
    """the hand-over between two decoder layers in one launch: the values of fnx_moe_combine followed by fnx_add_norm_q8"""
    rng = np.random.default_rng(806 + T)
    part = rng.standard_normal((T * topk, n)).astype(np.float32)
    topw = rng.random((T, topk)).astype(np.float32)
    sh, shl = rng.standard_normal((T, n)).astype(np.float32), rng.standard_normal(T).astype(np.float32)
    x, w = rng.standard_normal((T, n)).astype(np.float32) * 2, rng.standard_normal(n).astype(np.float32)
    comb = dev.moe_combine(part, topw, sh, shl)
    assert rel_l2(comb, oracle.moe_combine(part, topw, sh, shl)) <= 1e-6   # the sigmoid's expf is the device's
    x2, xn, xq = dev.combine_add_norm_q8(part, topw, sh, shl, x, w, 1e-6)
    want_x, want_n, want_q = dev.add_norm_q8(x, comb, w, 1e-6)
    assert int(np.count_nonzero(x2.view(np.uint32) != want_x.view(np.uint32))) == 0
    assert int(np.count_nonzero(xn.view(np.uint32) != want_n.view(np.uint32))) == 0
    assert int(np.count_nonzero(xq != want_q)) == 0


@pytest.mark.parametrize("rows,cols,T", [(37, 1024, 3), (1000, 2048, 16), (2048, 4096, 16), (513, 256, 5), (8192, 2048, 1),
                                         (151936, 2048, 16)])   # the last: benchmark config 4's output head
def test_q8s_gemv_bit_exact(dev, oracle, rows, cols, T):
    print(f"case q8s_gemv rows={rows} cols={cols} T={T}", flush=True)
    rng = np.random.default_rng(810 + rows)
    w = (rng.standard_normal((rows, cols)) * 0.05).astype(np.float32)
    q, d = np.zeros((rows, cols), dtype=np.int8), np.zeros((rows, cols // 32), dtype=np.uint16)
    oracle.lib.fnx_o_quantize_q8_0_split(ol.ptr(w), rows, cols, ol.ptr(q), ol.ptr(d))
    x = rng.standard_normal((T, cols)).astype(np.float32)
    yq = oracle.quantize_q8_1(x)
    want = np.zeros((T, rows), dtype=np.float32)
    oracle.lib.fnx_o_q8s_gemv(ol.ptr(q), ol.ptr(d), rows, cols, ol.ptr(yq), ol.ptr(want), rows, T)
    got = dev.q8s_gemv(q, d, yq, T)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert rel_l2(got, x.astype(np.float64) @ w.astype(np.float64).T) < 2e-2   # and it is the product it claims to be
    # the same values found elsewhere: the tile-major layout (fnx_q8s_tile), rows that do not fill the last tile included
    tiled = dev.q8s_gemv(q, d, yq, T, tiled=True)
    assert np.array_equal(tiled.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("rope", [ROPE, YARN])
@pytest.mark.parametrize("nq,nkv,T,pos0", [(4, 2, 3, 5), (16, 2, 16, 32000), (8, 1, 1, 0)])
def test_attn_prep_append(dev, oracle, nq, nkv, T, pos0, rope):
    print(f"case attn_prep nq={nq} nkv={nkv} T={T} pos0={pos0} scaled={rope[1]}", flush=True)
    rng = np.random.default_rng(820 + nq + T)
    qg = rng.standard_normal((T, nq, 512)).astype(np.float32)
    k, v = rng.standard_normal((T, nkv, 256)).astype(np.float32), rng.standard_normal((T, nkv, 256)).astype(np.float32)
    qn, kn = (1 + 0.1 * rng.standard_normal(256)).astype(np.float32), (1 + 0.1 * rng.standard_normal(256)).astype(np.float32)
    ctx = pos0 + T + 2
    kc0 = rng.integers(0, 1000, (ctx, nkv, 256)).astype(np.uint16)
    vc0 = rng.integers(0, 1000, (ctx, nkv, 256)).astype(np.uint16)
    kc, vc, q2, k2 = kc0.copy(), vc0.copy(), qg.copy(), k.copy()
    import ctypes as C
    r = td.RopeO(*rope)
    oracle.lib.fnx_o_attn_prep_append(ol.ptr(q2), ol.ptr(k2), ol.ptr(v), ol.ptr(qn), ol.ptr(kn), ol.ptr(kc), ol.ptr(vc), nq, nkv, 256, 64, T, pos0,
                                      1e-6, C.cast(C.pointer(r), C.c_void_p))
    gq, gk, gkc, gvc = dev.attn_prep_append(qg, k, v, qn, kn, kc0, vc0, nq, nkv, pos0, 1e-6, rope)
    # the angles are the same floats on both sides (the frequencies come from the host); sin, cos and rsqrt differ in the last bits
    dq, dk = float(np.abs(gq.reshape(q2.shape) - q2).max()), float(np.abs(gk.reshape(k2.shape) - k2).max())
    assert dq <= 2e-5 and dk <= 2e-5, (dq, dk)
    assert np.array_equal(gvc, vc), "v is only rounded to f16"
    dkc = float(np.abs(gkc.view(np.float16).astype(np.float32) - kc.view(np.float16).astype(np.float32)).max())
    assert dkc <= 4e-3, dkc   # one f16 step at magnitude 4
    assert np.array_equal(gkc[:pos0], kc0[:pos0]) and np.array_equal(gkc[pos0 + T:], kc0[pos0 + T:]), "only the window's rows are written"


@pytest.mark.parametrize("nq,nkv,T,pos0", [(4, 2, 3, 37), (16, 2, 16, 3000), (16, 2, 16, 0), (8, 1, 5, 511), (2, 2, 1, 64), (16, 2, 16, 1017), (16, 2, 7, 500),
                                           (16, 2, 16, 32752),   # benchmark config 4's window at the end of a 32,768-position cache
                                           # windows of few queries (up to 64 a kv head) run half a split a block: the last such row count,
                                           # the first that does not, a decode round's window at a long context, a context that ends in a second half
                                           (16, 2, 8, 700), (16, 2, 9, 700), (16, 2, 2, 32752), (16, 2, 4, 300)])
def test_attn_matches_oracle(dev, oracle, nq, nkv, T, pos0):
    print(f"case attn nq={nq} nkv={nkv} T={T} pos0={pos0}", flush=True)
    rng = np.random.default_rng(830 + nq + pos0)
    qg = rng.standard_normal((T, nq, 512)).astype(np.float32)
    kc = rng.standard_normal((pos0 + T + 3, nkv, 256)).astype(np.float16)
    vc = rng.standard_normal((pos0 + T + 3, nkv, 256)).astype(np.float16)
    kc[pos0 + T:], vc[pos0 + T:] = np.nan, np.inf   # cells past the window's rows must not be read into the result
    want = np.zeros((T, nq, 256), dtype=np.float32)
    oracle.lib.fnx_o_attn(ol.ptr(qg), ol.ptr(kc), ol.ptr(vc), ol.ptr(want), nq, nkv, 256, T, pos0)
    got = dev.attn(qg, kc, vc, nq, nkv, pos0)
    err = rel_l2(got, want)
    print("attention rel l2", err, flush=True)
    assert err <= 2e-5   # q and the probabilities are split into two f16 terms each: fp32-level agreement
    assert np.all(np.isfinite(got))


@pytest.mark.parametrize("max_ctx", [192, 520])
def test_attn_window_ends_at_the_caches_last_cell(dev, oracle, max_ctx):
    """a cache whose size is not a multiple of the split (512) or is smaller than one, the window's last row in the last
    cell: the largest position that is in range (positions out of range are a matter of the host-side bounds test)"""
    nq, nkv, T = 16, 2, 16
    pos0 = max_ctx - T
    print(f"case attn end of cache max_ctx={max_ctx} pos0={pos0}", flush=True)
    rng = np.random.default_rng(840 + max_ctx)
    qg = rng.standard_normal((T, nq, 512)).astype(np.float32)
    kc, vc = rng.standard_normal((max_ctx, nkv, 256)).astype(np.float16), rng.standard_normal((max_ctx, nkv, 256)).astype(np.float16)
    want = np.zeros((T, nq, 256), dtype=np.float32)
    oracle.lib.fnx_o_attn(ol.ptr(qg), ol.ptr(kc), ol.ptr(vc), ol.ptr(want), nq, nkv, 256, T, pos0)
    got = dev.attn(qg, kc, vc, nq, nkv, pos0)
    assert rel_l2(got, want) <= 2e-5


def chain_close(got, want, fresh):
    rows = [rel_l2(got[i], want[i]) for i in range(len(want))]
    assert max(rows) <= 1e-2, rows
    assert not fresh or min(rows) <= 1e-5, rows


@pytest.fixture(scope="module")
def model(oracle):
    return td.TinyDecoder(oracle, seed=11)


@pytest.mark.parametrize("tiled", [True, False])
def test_decoder_verify_and_draft(dev, oracle, model, tiled):
    """tiled: the dense matrices tile-major (fnx_q8s_tile) or as the reference's split layout"""
    o, d = td.OracleSession(model), fnx_gpu.DecoderDev(dev, model, tiled=tiled)
    pos = 0
    for toks in ([3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7, 9, 3], [2, 7, 18], [281]):
        print(f"case decoder_verify T={len(toks)} pos={pos}", flush=True)
        a, b = o.verify(toks, pos), d.verify(toks, pos)
        assert b["err"] == 0
        assert np.array_equal(a["best"], b["best"])
        chain_close(b["hidden"], a["hidden"], pos == 0)
        chain_close(b["logits"], a["logits"], pos == 0)
        nxt = toks[1:] + [int(a["best"][-1])]
        da, db = o.draft(a["hidden"], nxt, pos), d.draft(a["hidden"], nxt, pos)
        assert np.array_equal(da["best"], db["best"])
        chain_close(db["hidden"], da["hidden"], pos == 0)
        chain_close(db["logits"], da["logits"], pos == 0)
        pos += len(toks)
    for (ka, va), (kb, vb) in zip(o.caches + [o.mtp_cache], d.caches_numpy()):
        assert rel_l2(kb.view(np.float16)[:pos], ka.view(np.float16)[:pos]) <= REL_L2
        assert rel_l2(vb.view(np.float16)[:pos], va.view(np.float16)[:pos]) <= REL_L2


def test_draft_head_options(dev, oracle, model):
    """engine.cu:2130-2131: the draft head over the tokens [dv0, dv1) alone and the last row's penalty list, against the oracle's
    same call; the control without the list keeps the last row's own pick"""
    o, d = td.OracleSession(model), fnx_gpu.DecoderDev(dev, model)
    toks = [3, 1, 4, 1, 5, 9, 2, 6]
    a = o.verify(toks, 0)
    nxt = toks[1:] + [int(a["best"][-1])]
    dv = (96, 608)
    plain_o, plain_d = o.draft(a["hidden"], nxt, 0, dv=dv), d.draft(a["hidden"], nxt, 0, dv=dv)
    assert plain_d["err"] == 0 and plain_d["logits"].shape == (len(toks), dv[1] - dv[0])
    assert np.array_equal(plain_o["best"], plain_d["best"]) and all(dv[0] <= int(b) < dv[1] for b in plain_d["best"])
    chain_close(plain_d["logits"], plain_o["logits"], True)
    top = int(plain_o["best"][-1]) - dv[0]
    pen, par = (np.array([top, 7, -3, dv[1] - dv[0]]), np.array([3, 0, 1, 1])), (1.2, 0.5, 40.0)
    print("case mtp_draft with dv0, dv1 and a penalty list", flush=True)
    po, pd = o.draft(a["hidden"], nxt, 0, dv=dv, pen=pen, par=par), d.draft(a["hidden"], nxt, 0, dv=dv, pen=pen, par=par)
    assert pd["err"] == 0
    assert np.array_equal(po["best"], pd["best"]) and int(pd["best"][-1]) != dv[0] + top
    chain_close(pd["logits"], po["logits"], True)
    # the list changed one value of the last row and nothing else
    changed = np.argwhere(pd["logits"] != plain_d["logits"])
    assert changed.tolist() == [[len(toks) - 1, top]]
    # a head whose row count is not dv1 - dv0 is refused before any launch
    M = type(d.M).from_buffer_copy(d.M)
    M.dv0, M.dv1 = 0, 10
    tok = dev.up(np.asarray(nxt, dtype=np.int32))
    src = dev.up(a["hidden"])
    assert dev.lib.fnx_mtp_draft(C.byref(d.D), C.byref(M), src.data_ptr(), tok.data_ptr(), len(nxt), d.pos.data_ptr(), C.byref(d.ws), dev.st()) != 0


def same_until_near_tie(oracle, model, prompt, a, b):
    """tokens a and b agree up to index i; at i the oracle's logits of the two candidates must be a near-tie (the chain's
    re-quantisation noise is ~2e-3 of a row's spread). Returns the agreed length."""
    i = next((j for j in range(min(len(a), len(b))) if a[j] != b[j]), min(len(a), len(b)))
    if i == min(len(a), len(b)):
        return i
    sess = td.OracleSession(model)
    seq = list(prompt) + list(a[:i])
    pos, r = 0, None
    for j in range(0, len(seq), 16):
        r = sess.verify(seq[j:j + 16], pos)
        pos += len(seq[j:j + 16])
    row = r["logits"][-1]
    gap = abs(float(row[a[i]]) - float(row[b[i]]))
    print(f"outputs part at {i}: {a[i]} vs {b[i]}, logit gap {gap:.2e}, row spread {float(row.std()):.2e}", flush=True)
    assert gap <= 2e-2 * float(row.std()), "the two candidates are not a near-tie: a real disagreement"
    assert max(float(row[a[i]]), float(row[b[i]])) >= float(row.max()) - gap - 1e-6
    return i


def test_speculative_rounds_emit_the_greedy_tokens(dev, oracle, model):
    # a prompt with repeats (so prompt lookup fires) decoded three ways: device speculative, oracle speculative, device plain greedy
    rng = np.random.default_rng(12)
    base = [int(t) for t in rng.integers(0, 1000, 12)]
    prompt = base + base[:7] + [int(t) for t in rng.integers(0, 1000, 3)] + base[2:6]

    def lookup_dev(ctx, lk, d1):
        return dev.lookup(np.asarray(ctx, dtype=np.int32), lk, d1)

    def lookup_cpu(ctx, lk, d1):
        return oracle.lookup_drafts(np.asarray(ctx, dtype=np.int32), lk, d1)

    out_d, rounds_d = td.spec_generate(fnx_gpu.DecoderDev(dev, model), lookup_dev, lambda r, o: dev.accept(r, o), prompt, 40)
    out_o, rounds_o = td.spec_generate(td.OracleSession(model), lookup_cpu, lambda r, o: oracle.accept_greedy(r, o), prompt, 40)
    out_g, rounds_g = td.spec_generate(fnx_gpu.DecoderDev(dev, model), lookup_dev, lambda r, o: dev.accept(r, o), prompt, 40, speculate=False)
    print("rounds", rounds_d, flush=True)
    assert out_d == out_g, "speculation does not change the greedy output (fnx_run.cpp:1198-1238)"
    same = same_until_near_tie(oracle, model, prompt, out_d, out_o)
    assert same >= 8, "device and oracle emit the same tokens (up to a near-tie of two logits, checked on the oracle's logits)"
    if same == len(out_o):
        assert rounds_d == rounds_o, "and take the same drafts and accepted lengths every round"
    # drafts from outside: the true continuation with 30% of the tokens corrupted, up to 15 a round. Several rows stand
    # per round, rejected rows' cache cells are overwritten by the next window, and the output is still the greedy one
    crng = np.random.default_rng(13)

    def forced(m, d1):
        k = int(crng.integers(1, 16))
        return [t if crng.random() > 0.3 else int(crng.integers(0, 1000)) for t in out_g[m:m + k]]

    crng_o = np.random.default_rng(13)

    def forced_o(m, d1):
        k = int(crng_o.integers(1, 16))
        return [t if crng_o.random() > 0.3 else int(crng_o.integers(0, 1000)) for t in out_g[m:m + k]]

    out_f, rounds_f = td.spec_generate(fnx_gpu.DecoderDev(dev, model), lookup_dev, lambda r, o: dev.accept(r, o), prompt, 40, forced=forced)
    out_fo, rounds_fo = td.spec_generate(td.OracleSession(model), lookup_cpu, lambda r, o: oracle.accept_greedy(r, o), prompt, 40, forced=forced_o)
    print("forced rounds", rounds_f, flush=True)
    assert out_f == out_g, "any drafts leave the device's output as it is"
    assert out_fo == out_o, "and the oracle's"
    if out_o == out_g:
        assert rounds_f == rounds_fo
    assert len(rounds_f) < len(rounds_g) and max(u for _, u in rounds_f) > 2

"""Pins for the oracle's composite functions (the MoE verify layer, one decoder layer, the decoder window and the draft
layer): each is compared with the same wiring written out here in numpy f64 over operands that the oracle's separately
pinned leaf functions produce (q8_1 rows, dequantised weights). Every comparison comes with controls: the same numpy
model with one wiring mistake (a norm taken from the wrong tensor, a residual left out, gate and up exchanged, the
shared expert dropped) must miss the oracle by far more than the tolerance, so the tolerance separates right from wrong.

The tolerance is not float rounding: h = silu(g) * u is rounded to q8_1 between the two mat-vecs, and a g or u that
differs in its last bit can move one rounded value by a whole step. 2e-3 of the result's norm covers that; the controls
miss by 3e-2 or more.

Wiring followed: engine.cu:1569-1757 (attention half, then the FFN half on the residual), engine.cu:2095-2133 (the draft
layer's input R = fc_hidden(rms(src) * norm_hid) + fc_embedding(rms(emb) * norm_emb), its own norm and head)."""
import numpy as np

import oracle_lib as ol
import tiny_decoder as td
from fnx_gpu import random_iq3s

TOL = 2e-3
MISS = 3e-2


def rel(a, b):
    return float(np.linalg.norm(np.asarray(a, dtype=np.float64) - b) / np.linalg.norm(b))


def q8_1_values(oracle, x):
    """the values a q8_1 row stands for: d * q per block of 32"""
    rows, n = x.shape
    b = oracle.quantize_q8_1(x).reshape(rows, n // 32, 36)
    d = b[:, :, :2].copy().view(np.float16).astype(np.float64)
    q = b[:, :, 4:].view(np.int8).astype(np.float64)
    return (q * d).reshape(rows, n)


def q8s_values(t):
    q, d = t
    return (q.reshape(q.shape[0], -1, 32).astype(np.float64) * d.view(np.float16).astype(np.float64)[:, :, None]).reshape(q.shape)


def dense(oracle, t, x):
    return q8_1_values(oracle, np.asarray(x, dtype=np.float32)) @ q8s_values(t).T


def rms(x, w, eps=1e-6):
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * w


def iq3s_matrix(oracle, blocks, rows, cols):
    return oracle.iq3s_dequant(blocks).astype(np.float64).reshape(rows, cols)


# ---------------------------------------------------------------- the MoE verify layer
def np_moe_layer(oracle, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x, wrong=None, sh_q8=None):
    T = x.shape[0]
    logits = oracle.gemv_f32(router, x)
    topi, topw = oracle.topk_logits(logits, nexp, topk)
    xv = q8_1_values(oracle, x)
    gs, ds = 2 * ff * n // 256 * 110, n * ff // 256 * 110

    def ffn(Wgu, Wd, row):
        gu_row = Wgu @ row
        g, u = (gu_row[:ff], gu_row[ff:]) if wrong != "gate_up" else (gu_row[ff:], gu_row[:ff])
        h = (g / (1 + np.exp(-g)) * u).astype(np.float32)
        return Wd @ q8_1_values(oracle, h[None, :])[0]

    out = np.zeros((T, n))
    for t in range(T):
        for k in range(topk):
            e = int(topi[t, k])
            out[t] += float(topw[t, k]) * ffn(iq3s_matrix(oracle, gu[e * gs:(e + 1) * gs], 2 * ff, n),
                                              iq3s_matrix(oracle, down[e * ds:(e + 1) * ds], n, ff), xv[t])
        if wrong != "no_shared":
            gate = 1 / (1 + np.exp(-float(logits[t, nexp]))) if wrong != "shared_ungated" else 1.0
            if sh_q8 is not None:
                out[t] += gate * ffn(q8s_values(sh_q8[0]), q8s_values(sh_q8[1]), xv[t])
            else:
                out[t] += gate * ffn(iq3s_matrix(oracle, sh_gu, 2 * ff, n), iq3s_matrix(oracle, sh_down, n, ff), xv[t])
    return out, logits, topi, topw


def test_moe_verify_layer_equals_its_parts(oracle):
    rng = np.random.default_rng(21)
    n, ff, nexp, topk, T = 256, 256, 8, 3, 5
    nb = lambda rows, cols: rows * cols // 256
    gu, down = random_iq3s(rng, nexp * nb(2 * ff, n), dmax=2e-2), random_iq3s(rng, nexp * nb(n, ff), dmax=2e-2)
    sh_gu, sh_down = random_iq3s(rng, nb(2 * ff, n), dmax=2e-2), random_iq3s(rng, nb(n, ff), dmax=2e-2)
    router = (rng.standard_normal((nexp + 1, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((T, n)).astype(np.float32)
    r = oracle.moe_verify_layer(n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x)
    want, logits, topi, topw = np_moe_layer(oracle, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x)
    assert np.array_equal(r["logits"], logits) and np.array_equal(r["topi"], topi) and np.array_equal(r["topw"], topw)
    assert rel(r["out"], want) <= TOL
    # the weights of a row: softmax over the picked logits (sum to one, ordered as the logits are)
    assert np.allclose(topw.sum(axis=1), 1.0, atol=1e-6)
    pl = np.take_along_axis(logits[:, :nexp], topi, axis=1).astype(np.float64)
    e = np.exp(pl - pl.max(axis=1, keepdims=True))
    assert np.allclose(topw, e / e.sum(axis=1, keepdims=True), rtol=1e-5)
    assert r["njobs"] == len(np.unique(topi))
    for wrong in ("gate_up", "no_shared", "shared_ungated"):
        bad = np_moe_layer(oracle, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x, wrong=wrong)[0]
        assert rel(r["out"], bad) >= MISS, wrong


def test_moe_verify_layer_with_a_q8_0_shared_expert(oracle):
    # engine.cu:1600-1604: the shared expert as dense split Q8_0 (q8s_gemv -> swiglu_stacked_q8_1 -> q8s_gemv)
    rng = np.random.default_rng(22)
    n, ff, nexp, topk, T = 256, 256, 8, 3, 5
    nb = lambda rows, cols: rows * cols // 256
    gu, down = random_iq3s(rng, nexp * nb(2 * ff, n), dmax=2e-2), random_iq3s(rng, nexp * nb(n, ff), dmax=2e-2)

    def q8(rows, cols):
        w = (rng.standard_normal((rows, cols)) * 2.0).astype(np.float32)
        q, d = np.zeros((rows, cols), dtype=np.int8), np.zeros((rows, cols // 32), dtype=np.uint16)
        oracle.lib.fnx_o_quantize_q8_0_split(ol.ptr(w), rows, cols, ol.ptr(q), ol.ptr(d))
        return q, d

    sh_q8 = (q8(2 * ff, n), q8(n, ff))
    router = (rng.standard_normal((nexp + 1, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((T, n)).astype(np.float32)
    r = oracle.moe_verify_layer(n, ff, nexp, topk, router, gu, down, None, None, x, sh_q8=sh_q8)
    want = np_moe_layer(oracle, n, ff, nexp, topk, router, gu, down, None, None, x, sh_q8=sh_q8)[0]
    assert rel(r["out"], want) <= TOL
    for wrong in ("gate_up", "no_shared", "shared_ungated"):
        bad = np_moe_layer(oracle, n, ff, nexp, topk, router, gu, down, None, None, x, wrong=wrong, sh_q8=sh_q8)[0]
        assert rel(r["out"], bad) >= MISS, wrong


# ---------------------------------------------------------------- a decoder layer, the window, the draft layer
def np_rope(y, pos, rope):
    base = rope[0]
    assert not rope[1]
    i = np.arange(32)
    th = pos * (base ** (-2.0 * i / 64))
    x0, x1 = y[:32].copy(), y[32:64].copy()
    y = y.copy()
    y[:32], y[32:64] = x0 * np.cos(th) - x1 * np.sin(th), x0 * np.sin(th) + x1 * np.cos(th)
    return y


class NpDecoder:
    """the tiny decoder in numpy f64; caches are kept as f16 values, as the device and the oracle keep them"""

    def __init__(self, m, wrong=None):
        self.m, self.o, self.c, self.wrong = m, m.oracle, m.cfg, wrong
        mk = lambda: (np.zeros((self.c["max_ctx"], self.c["nkv"], 256)), np.zeros((self.c["max_ctx"], self.c["nkv"], 256)))
        self.caches = [mk() for _ in m.layers]
        self.mtp_cache = mk()

    def layer(self, L, cache, x, pos0):
        c, o, wrong = self.c, self.o, self.wrong
        nq, nkv, T = c["nq"], c["nkv"], x.shape[0]
        kc, vc = cache
        xn = rms(x, L["attn_norm"] if wrong != "layer_norms" else L["ffn_norm"])
        qg = dense(o, L["wq"], xn).reshape(T, nq, 512)
        k = dense(o, L["wk"], xn).reshape(T, nkv, 256)
        v = dense(o, L["wv"], xn).reshape(T, nkv, 256)
        att = np.zeros((T, nq, 256))
        for t in range(T):
            for h in range(nkv):
                kc[pos0 + t, h] = np_rope(rms(k[t, h], L["k_norm"]), pos0 + t, self.m.rope).astype(np.float32).astype(np.float16)
                vc[pos0 + t, h] = v[t, h].astype(np.float32).astype(np.float16)
        for t in range(T):
            ctx = pos0 + t + 1 if wrong != "not_causal" else pos0 + T
            for h in range(nq):
                kv = h // (nq // nkv)
                q = np_rope(rms(qg[t, h, :256], L["q_norm"]), pos0 + t, self.m.rope)
                s = kc[:ctx, kv] @ q / 16.0
                p = np.exp(s - s.max())
                att[t, h] = (p / p.sum()) @ vc[:ctx, kv] / (1 + np.exp(-qg[t, h, 256:]))
        a = dense(o, L["wo"], att.reshape(T, nq * 256))
        x = x + a if wrong != "no_attn_residual" else a
        ffn_norm = L["ffn_norm"] if wrong != "layer_norms" else L["attn_norm"]
        xn = rms(x, ffn_norm if wrong != "ffn_norm_flat" else 1.0).astype(np.float32)
        f = o.moe_verify_layer(c["n"], c["ff"], c["nexp"], c["topk"], L["router"], L["gu"], L["down"], L["sh_gu"], L["sh_down"], xn)["out"]
        return x + f if wrong != "no_ffn_residual" else f.astype(np.float64)

    def head(self, norm, head, x):
        return dense(self.o, head, rms(x, norm))

    def verify(self, tokens, pos0):
        x = self.m.emb[np.asarray(tokens)].astype(np.float64)
        for L, cache in zip(self.m.layers, self.caches):
            x = self.layer(L, cache, x, pos0)
        return dict(hidden=x, logits=self.head(self.m.out_norm, self.m.head, x))

    def draft(self, src, tokens, pos0):
        M, o = self.m.mtp, self.o
        nh, ne = (M["norm_hid"], M["norm_emb"]) if self.wrong != "mtp_norms" else (M["norm_emb"], M["norm_hid"])
        fh, fe = (M["fc_hid"], M["fc_emb"]) if self.wrong != "mtp_fc" else (M["fc_emb"], M["fc_hid"])
        x = dense(o, fh, rms(src, nh))
        if self.wrong != "mtp_no_emb":
            x = x + dense(o, fe, rms(self.m.emb[np.asarray(tokens)].astype(np.float64), ne))
        x = self.layer(M["layer"], self.mtp_cache, x, pos0)
        norm = M["out_norm"] if self.wrong != "mtp_head_norm" else self.m.out_norm
        return dict(hidden=x, logits=self.head(norm, M["head"], x))


def check_best(best, logits):
    """the oracle's pick is the row's maximum wherever the numpy logits have a clear one"""
    for t in range(len(best)):
        s = np.sort(logits[t])
        if s[-1] - s[-2] > 1e-3 * max(1.0, abs(s[-1])):
            assert int(best[t]) == int(np.argmax(logits[t]))


TOKS = [7, 11, 400, 23, 999, 5, 42, 77]


def test_decoder_window_equals_its_wiring(oracle):
    m = td.TinyDecoder(oracle, seed=31)
    sess, mine = td.OracleSession(m), NpDecoder(m)
    # two windows, so the second reads cells the first wrote
    for pos0, toks in ((0, TOKS[:5]), (5, TOKS[5:])):
        got, want = sess.verify(toks, pos0), mine.verify(toks, pos0)
        assert rel(got["hidden"], want["hidden"]) <= TOL
        assert rel(got["logits"], want["logits"]) <= TOL
        check_best(got["best"], want["logits"])
    for (kc, vc), (nk, nv) in zip(sess.caches, mine.caches):
        assert rel(kc.view(np.float16)[:8], nk[:8]) <= TOL and rel(vc.view(np.float16)[:8], nv[:8]) <= TOL
        assert not kc[8:].any() and not vc[8:].any()
    for wrong in ("layer_norms", "no_attn_residual", "no_ffn_residual", "not_causal"):
        bad, s2 = NpDecoder(m, wrong), td.OracleSession(m)
        assert rel(s2.verify(TOKS[:5], 0)["hidden"], bad.verify(TOKS[:5], 0)["hidden"]) >= MISS, wrong
    # the FFN half adds a tenth of the residual's norm in this model, so a mistake inside it alone shows less: five times TOL
    assert rel(td.OracleSession(m).verify(TOKS[:5], 0)["hidden"], NpDecoder(m, "ffn_norm_flat").verify(TOKS[:5], 0)["hidden"]) >= 5 * TOL


def test_single_layer_step_by_step(oracle):
    # one layer alone (a one-layer model), token by token through the cache: T = 1 windows at growing positions
    m = td.TinyDecoder(oracle, seed=32, nlayers=1)
    sess, mine = td.OracleSession(m), NpDecoder(m)
    for p, tok in enumerate(TOKS[:4]):
        got, want = sess.verify([tok], p), mine.verify([tok], p)
        assert rel(got["hidden"], want["hidden"]) <= TOL


def test_mtp_draft_equals_its_wiring(oracle):
    m = td.TinyDecoder(oracle, seed=33)
    sess, mine = td.OracleSession(m), NpDecoder(m)
    src = sess.verify(TOKS[:6], 0)["hidden"]
    nxt = TOKS[1:7]
    for pos0, rows in ((0, slice(0, 4)), (4, slice(4, 6))):
        got, want = sess.draft(src[rows], nxt[rows], pos0), mine.draft(src[rows], nxt[rows], pos0)
        assert rel(got["hidden"], want["hidden"]) <= TOL
        assert rel(got["logits"], want["logits"]) <= TOL
        check_best(got["best"], want["logits"])
    # the draft layer keeps its own cache: the main layers' cells are untouched by it
    assert rel(sess.mtp_cache[0].view(np.float16)[:6], mine.mtp_cache[0][:6]) <= TOL
    for wrong in ("mtp_norms", "mtp_fc", "mtp_no_emb", "mtp_head_norm", "no_attn_residual", "no_ffn_residual"):
        bad, s2 = NpDecoder(m, wrong), td.OracleSession(m)
        got, miss = s2.draft(src[:4], nxt[:4], 0), bad.draft(src[:4], nxt[:4], 0)
        which = "logits" if wrong == "mtp_head_norm" else "hidden"
        assert rel(got[which], miss[which]) >= MISS, wrong


def test_mtp_draft_head_options_equal_their_wiring(oracle):
    """engine.cu:2130-2131: a head of the tokens [dv0, dv1) alone gives those logits and token ids from dv0; the penalty list
    touches the last row only, before its pick. Control: the same call without the list keeps the row's unpenalised pick."""
    m = td.TinyDecoder(oracle, seed=33)
    src = td.OracleSession(m).verify(TOKS[:6], 0)["hidden"]
    nxt = TOKS[1:7]
    full = NpDecoder(m).draft(src[:4], nxt[:4], 0)["logits"]
    dv0, dv1 = 200, 700
    part = full[:, dv0:dv1]
    top = int(np.argmax(part[3]))
    # the row's top token (counted twice), a token whose count is zero (skipped), and indexes outside the head (skipped)
    idx, cnt = np.array([top, 5, -1, dv1 - dv0]), np.array([2, 0, 1, 1])
    par = (1.3, 0.25, 50.0)
    want = part.copy()
    l = want[3, top]
    want[3, top] = (l * par[0] if l <= 0 else l / par[0]) - 2 * par[1] - par[2]
    got = td.OracleSession(m).draft(src[:4], nxt[:4], 0, dv=(dv0, dv1), pen=(idx, cnt), par=par)
    assert got["logits"].shape == (4, dv1 - dv0)
    assert rel(got["logits"], want) <= TOL
    assert rel(got["logits"][3, top], want[3, top]) <= TOL and got["logits"][3, 5] == td.OracleSession(m).draft(src[:4], nxt[:4], 0, dv=(dv0, dv1))["logits"][3, 5]
    assert all(dv0 <= int(b) < dv1 for b in got["best"])
    check_best(got["best"] - dv0, want)
    assert int(got["best"][3]) != dv0 + top, "the penalised token lost the row"
    ctl = td.OracleSession(m).draft(src[:4], nxt[:4], 0, dv=(dv0, dv1))
    assert rel(ctl["logits"], part) <= TOL and int(ctl["best"][3]) == dv0 + top
    assert np.array_equal(ctl["best"][:3], got["best"][:3]), "rows before the last are not penalised"
    # the whole vocabulary (dv0 = dv1 = 0) with a list: the same row rule
    whole = td.OracleSession(m).draft(src[:4], nxt[:4], 0, pen=(np.array([int(np.argmax(full[3]))]), np.array([1])), par=par)
    assert int(whole["best"][3]) != int(np.argmax(full[3])) and np.array_equal(whole["logits"][:3], td.OracleSession(m).draft(src[:4], nxt[:4], 0)["logits"][:3])

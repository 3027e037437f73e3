"""The committed vectors (tests/golden/verify_path.npz, made by tests/golden/make_fixtures.py; sampler_path.npz, made by
tests/golden/make_sampler_fixtures.py) against the oracle (CPU), the library's host functions (CPU) and the device
library (GPU)."""
import os

import numpy as np
import pytest

import fnx_gpu
from fnx_gpu import JOB_DTYPE

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "verify_path.npz"))


def test_oracle_reproduces_the_fixtures(oracle):
    assert np.array_equal(oracle.iq3s_dequant(G["blocks2"]), G["blocks2_decoded"])
    assert np.array_equal(oracle.quantize_q8_1(G["x3"]), G["x3_q8_1"])
    assert np.array_equal(oracle.gemv_iq3s(G["w64x512"], 64, 512, G["x3"]), G["y3"])
    topi, topw = oracle.topk_logits(G["logits"], 512, 10)
    assert np.array_equal(topi, G["topi"]) and np.array_equal(topw, G["topw"])
    gu, dn = oracle.jobs(topi)
    assert np.array_equal(gu.view(np.uint8).reshape(len(gu), -1), G["jobs_gu"])
    assert np.array_equal(oracle.gemv_f32(G["router_w"], G["router_x"]), G["router_y"])
    assert np.array_equal(oracle.swiglu_stacked_q8_1(G["swiglu_gu"], 32), G["swiglu_hq"])
    assert np.array_equal(oracle.moe_combine(G["comb_part"], G["comb_topw"], G["comb_sh"], G["comb_shl"]), G["comb_out"])
    bv, bi, err = oracle.argmax(G["argmax_logits"], v0=11)
    assert np.array_equal(bi, G["argmax_i"]) and err == int(G["argmax_err"][0]) == 16
    for i in range(20):
        c = G["lk_ctx"][G["lk_off"][i]:G["lk_off"][i + 1]]
        lk, d1, m = (int(v) for v in G["lk_params"][i])
        d, mm = oracle.lookup_drafts(c, lk, d1)
        assert list(d) == list(G["lk_drafts"][G["lk_doff"][i]:G["lk_doff"][i + 1]]) and mm == m
    for i in range(12):
        assert oracle.accept_greedy(G["acc_rows"][i], G["acc_o"][i]) == int(G["acc_n"][i])


@pytest.mark.gpu
def test_device_reproduces_the_fixtures():
    dev = fnx_gpu.Dev()
    assert np.array_equal(dev.quantize_q8_1(G["x3"]), G["x3_q8_1"])
    for packed in (False, True):
        y = dev.gemv_iq3s(G["w64x512"], 64, 512, G["x3"], packed=packed)
        assert np.linalg.norm(y - G["y3"]) <= 1e-5 * np.linalg.norm(G["y3"])
    r = dev.route(G["logits"], 512, 10)
    assert np.array_equal(r["topi"], G["topi"]) and np.array_equal(r["topw"].view(np.uint32), G["topw"].view(np.uint32))
    want = np.ascontiguousarray(G["jobs_gu"]).reshape(-1).view(JOB_DTYPE)
    assert len(r["gu"]) == len(want)
    for g, w in zip(r["gu"], want):
        n = int(w["n"])
        assert int(g["w"]) == int(w["w"]) and int(g["n"]) == n
        assert np.array_equal(g["y"][:n], w["y"][:n]) and np.array_equal(g["out"][:n], w["out"][:n])
    assert np.array_equal(dev.gemv(G["router_w"], G["router_x"]), G["router_y"])
    bv, bi, err = dev.argmax(G["argmax_logits"], v0=11)
    assert np.array_equal(bi, G["argmax_i"]) and err == 16
    for i in range(20):
        c = G["lk_ctx"][G["lk_off"][i]:G["lk_off"][i + 1]]
        lk, d1, m = (int(v) for v in G["lk_params"][i])
        d, mm = dev.lookup(c, lk, d1)
        assert list(d) == list(G["lk_drafts"][G["lk_doff"][i]:G["lk_doff"][i + 1]]) and mm == m
    for i in range(12):
        assert dev.accept(G["acc_rows"][i], G["acc_o"][i]) == int(G["acc_n"][i])


S = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sampler_path.npz"))


def sampler_lists():
    """the fixture's penalty and bias lists as test_oracle_sampler's helpers take them"""
    pen = [[(int(S["tk_pen_tok"][t, i]), int(S["tk_pen_cnt"][t, i])) for i in range(int(S["tk_pen_n"][t]))] for t in range(3)]
    par = [tuple(float(v) for v in S["tk_par"][t]) for t in range(3)]
    off = np.concatenate([[0], np.cumsum(S["tk_bias_n"])])
    bias = [[(int(S["tk_bias_tok"][i]), float(S["tk_bias_val"][i])) for i in range(off[t], off[t + 1])] for t in range(3)]
    return pen, par, bias


def test_oracle_and_host_sampler_reproduce_the_fixtures(oracle):
    import ctypes as C
    from test_oracle_sampler import o_accept, o_dist, o_top_tokens
    pen, par, bias = sampler_lists()
    ov, oi, L, err = o_top_tokens(oracle, S["tk_logits"], v0=100, pen=pen, par=par, bias=bias)
    assert np.array_equal(oi, S["tk_out_i"]) and np.array_equal(ov.view(np.uint32), S["tk_out_v"].view(np.uint32))
    assert np.array_equal(L.view(np.uint32), S["tk_logits_after"].view(np.uint32)) and err == int(S["tk_err"][0]) == 16
    t, top_p, min_p, top_k = (float(v) for v in S["sp_params"])
    kw = dict(temperature=t, top_p=top_p, min_p=min_p, top_k=int(top_k))
    ids, p = o_dist(oracle, S["tk_out_v"][0], S["tk_out_i"][0], **kw)
    assert np.array_equal(ids, S["dist_ids"]) and np.array_equal(p, S["dist_p"])
    pkg = fnx_gpu.package()
    lib = pkg.lib()
    s = pkg.Sampling(t, top_p, min_p, int(top_k))
    hi, hp = np.zeros(64, np.int32), np.zeros(64, np.float64)
    cv, ci = np.ascontiguousarray(S["tk_out_v"][:2]), np.ascontiguousarray(S["tk_out_i"][:2])
    k = lib.fnx_make_dist(cv.ctypes.data, ci.ctypes.data, 64, C.byref(s), hi.ctypes.data, hp.ctypes.data)
    assert k == len(S["dist_ids"]) and np.array_equal(hi[:k], S["dist_ids"]) and np.array_equal(hp[:k], S["dist_p"])
    rows = np.ascontiguousarray(S["sp_rows"])
    for i in range(8):
        n, o, used = o_accept(oracle, cv, ci, rows, S["sp_u"][i], **kw)
        want = (int(S["sp_n"][i]), [int(v) for v in S["sp_o"][i][:int(S["sp_n"][i])]], int(S["sp_used"][i]))
        assert (n, o, used) == want
        ho, hu = np.zeros(2, np.int32), C.c_int()
        u = np.ascontiguousarray(S["sp_u"][i])
        hn = lib.fnx_accept_sampled(cv.ctypes.data, ci.ctypes.data, 64, 2, rows.ctypes.data, C.byref(s), None, None, None, 1, u.ctypes.data, 3,
                                    ho.ctypes.data, C.byref(hu))
        assert (hn, [int(v) for v in ho[:hn]], hu.value) == want


@pytest.mark.gpu
def test_device_reproduces_the_sampler_fixtures():
    from test_gpu_sampler import d_top_tokens
    dev = fnx_gpu.Dev()
    pen, par, bias = sampler_lists()
    ov, oi, L, err = d_top_tokens(dev, S["tk_logits"], v0=100, pen=pen, par=par, bias=bias)
    assert np.array_equal(oi, S["tk_out_i"]) and np.array_equal(ov.view(np.uint32), S["tk_out_v"].view(np.uint32))
    assert np.array_equal(L.view(np.uint32), S["tk_logits_after"].view(np.uint32)) and err == 16

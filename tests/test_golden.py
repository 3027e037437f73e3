"""The committed vectors (tests/golden/verify_path.npz, made by tests/golden/make_fixtures.py) against the oracle
(CPU) and against the device library (GPU)."""
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
    assert np.array_equal(r["topi"], G["topi"]) and np.allclose(r["topw"], G["topw"], rtol=2e-6, atol=0)
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

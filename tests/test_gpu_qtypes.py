"""The other expert types the operators take (kernels.cu:2454-2471: Q4_0, Q8_0, IQ4_NL, Q4_K, Q5_K here) through
fnx_mmvq / fnx_moe_gate_up / fnx_moe_down against the CPU oracle. Bar: relative L2 <= 1e-6 (the same per-sub-block terms,
the same order of sums; what is left is the compiler's choice among equal-valued float forms)."""
import ctypes as C

import numpy as np
import pytest

import fnx_gpu
import oracle_lib as ol
import qtype_blocks as qb
from fnx_gpu import JOB_DTYPE

pytestmark = pytest.mark.gpu
TYPES = [qb.Q4_0, qb.Q5_1, qb.Q8_0, qb.IQ4_NL, qb.IQ4_XS, qb.Q4_K, qb.Q5_K]


def rel_l2(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return fnx_gpu.Dev()


def make_jobs(rng, nexp, njobs, nrows_y):
    jobs = np.zeros(njobs, dtype=JOB_DTYPE)
    out_row = 0
    for j in range(njobs):
        n = int(rng.integers(1, 17)) if j else 16
        jobs["w"][j] = int(rng.integers(0, nexp))
        jobs["n"][j] = n
        jobs["y"][j, :n] = rng.integers(0, nrows_y, n)
        jobs["out"][j, :n] = np.arange(out_row, out_row + n)
        out_row += n
    return jobs, out_row


@pytest.mark.parametrize("qtype", TYPES)
@pytest.mark.parametrize("nrows,ncols", [(64, 512), (30, 2048), (8, 4096)])
def test_mmvq_other_types(dev, oracle, qtype, nrows, ncols):
    print(f"case mmvq type={qtype} {nrows} x {ncols}", flush=True)
    rng = np.random.default_rng(1000 * qtype + nrows)
    values, nbytes = qb.SHAPE[qtype]
    nexp, row_bytes = 3, ncols // values * nbytes
    w = qb.random_blocks(rng, qtype, nexp * nrows * ncols // values)
    x = rng.standard_normal((20, ncols)).astype(np.float32)
    yq = oracle.quantize_q8_1(x)
    jobs, out_rows = make_jobs(rng, nexp, 5, 20)
    want = np.zeros((out_rows, nrows), np.float32)
    oracle.lib.fnx_o_mmvq_type(qtype, ol.ptr(w), nrows * row_bytes, nrows, ncols, ol.ptr(np.ascontiguousarray(jobs)), len(jobs), ol.ptr(yq), ol.ptr(want),
                               nrows, 8)
    t = dev.torch
    dw_, dj, dy = dev.up(w), dev.up(jobs.view(np.uint8).reshape(-1)), dev.up(yq)
    out = dev.zeros((out_rows, nrows), t.float32)
    W = dev.pkg.DW(dw_.data_ptr(), qtype, ncols, nrows, row_bytes, None)
    nj = dev.up(np.array([len(jobs)], dtype=np.int32))
    dev.ok(dev.lib.fnx_mmvq(C.byref(W), nrows * row_bytes, dj.data_ptr(), nj.data_ptr(), len(jobs), dy.data_ptr(), out.data_ptr(), nrows, dev.st()))
    dev.sync()
    err = rel_l2(out.cpu().numpy(), want)
    assert err <= 1e-6, err
    # against the decoded weights and the real activations: the q8_1 path's own error band (dense.cuh:258-259: ~6e-3)
    wd = qb.np_dequant(qtype, w).reshape(nexp, nrows, ncols).astype(np.float64)
    exact = np.concatenate([x[jobs["y"][j, :jobs["n"][j]]].astype(np.float64) @ wd[jobs["w"][j]].T for j in range(len(jobs))])
    assert rel_l2(out.cpu().numpy(), exact) <= 3e-2


def test_gate_up_and_down_with_q4_k_experts(dev, oracle):
    # the operators of a window's MoE half, one by one, on Q4_K experts: gate|up, SwiGLU -> q8_1 in the library's buffer, down
    rng = np.random.default_rng(4242)
    qtype, n, ff, nexp, T, topk = qb.Q4_K, 512, 256, 4, 3, 2
    values, nbytes = qb.SHAPE[qtype]
    gu_w = qb.random_blocks(rng, qtype, nexp * 2 * ff * n // values)
    dn_w = qb.random_blocks(rng, qtype, nexp * n * ff // values)
    x = rng.standard_normal((T, n)).astype(np.float32)
    xq = oracle.quantize_q8_1(x)
    topi = np.array([[0, 2], [2, 1], [3, 0]], np.int32)
    gu_jobs, dn_jobs = oracle.jobs(topi)
    P = T * topk
    print("case gate|up, down on Q4_K experts", flush=True)
    gu_rb, dn_rb = n // values * nbytes, ff // values * nbytes
    want_gu = np.zeros((P, 2 * ff), np.float32)
    oracle.lib.fnx_o_mmvq_type(qtype, ol.ptr(gu_w), 2 * ff * gu_rb, 2 * ff, n, ol.ptr(np.ascontiguousarray(gu_jobs)), len(gu_jobs), ol.ptr(xq), ol.ptr(want_gu),
                               2 * ff, 8)
    hq = oracle.swiglu_stacked_q8_1(want_gu, ff)
    want_part = np.zeros((P, n), np.float32)
    oracle.lib.fnx_o_mmvq_type(qtype, ol.ptr(dn_w), n * dn_rb, n, ff, ol.ptr(np.ascontiguousarray(dn_jobs)), len(dn_jobs), ol.ptr(hq), ol.ptr(want_part), n, 8)
    t = dev.torch
    dgu, ddn, dxq = dev.up(gu_w), dev.up(dn_w), dev.up(xq)
    jg, jd = dev.up(gu_jobs.view(np.uint8).reshape(-1)), dev.up(dn_jobs.view(np.uint8).reshape(-1))
    nj = dev.up(np.array([len(gu_jobs)], dtype=np.int32))
    gu, part = dev.zeros((P, 2 * ff), t.float32), dev.zeros((P, n), t.float32)
    A = dev.pkg.DW(dgu.data_ptr(), qtype, n, 2 * ff, gu_rb, None)
    B = dev.pkg.DW(ddn.data_ptr(), qtype, ff, n, dn_rb, None)
    dev.ok(dev.lib.fnx_moe_gate_up(C.byref(A), 2 * ff * gu_rb, jg.data_ptr(), nj.data_ptr(), P, dxq.data_ptr(), gu.data_ptr(), topk, dev.st()))
    dev.ok(dev.lib.fnx_moe_down(C.byref(B), n * dn_rb, jd.data_ptr(), nj.data_ptr(), P, gu.data_ptr(), part.data_ptr(), dev.st()))
    dev.sync()
    assert rel_l2(gu.cpu().numpy(), want_gu) <= 1e-6
    assert rel_l2(part.cpu().numpy(), want_part) <= 1e-3   # SwiGLU's expf moves an int8 code by one step now and then

"""The oracle's decoders and dots for the other expert types (Q4_0, Q8_0, IQ4_NL, Q4_K, Q5_K): the decoders against the
reference's own conv::dequantize (oracle/_ref) and numpy restatements of the layouts, bit for bit; a sub-block's dot
against the decoded weights times the q8_1 values in f64."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as ol
import qtype_blocks as qb

TYPES = [qb.Q4_0, qb.Q5_1, qb.Q8_0, qb.IQ4_NL, qb.IQ4_XS, qb.Q4_K, qb.Q5_K]


def o_dequant(oracle, qtype, blocks):
    values, nbytes = qb.SHAPE[qtype]
    n = blocks.size // nbytes * values
    y = np.zeros(n, np.float32)
    oracle.lib.fnx_o_dequant(qtype, ol.ptr(blocks), n, ol.ptr(y))
    return y


@pytest.mark.parametrize("qtype", TYPES)
def test_decoders_equal_numpy(oracle, qtype):
    rng = np.random.default_rng(40 + qtype)
    blocks = qb.random_blocks(rng, qtype, 24)
    got, want = o_dequant(oracle, qtype, blocks), qb.np_dequant(qtype, blocks)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    values, nbytes = C.c_int(), C.c_int()
    assert oracle.lib.fnx_o_type_block(qtype, C.byref(values), C.byref(nbytes)) == 0 and (values.value, nbytes.value) == qb.SHAPE[qtype]


@pytest.mark.parametrize("qtype", [t for t in TYPES if t != qb.Q5_1])   # the reference's host code has no Q5_1 dequantiser
def test_decoders_equal_the_reference(oracle, ref, qtype):
    rng = np.random.default_rng(50 + qtype)
    blocks = qb.random_blocks(rng, qtype, 64)
    got = o_dequant(oracle, qtype, blocks)
    want = np.zeros_like(got)
    assert ref.fnx_ref_dequantize(qtype, ol.ptr(blocks), got.size, ol.ptr(want)) == 0
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "tensor_convert.hpp:152-265"


@pytest.mark.parametrize("qtype", TYPES)
def test_sub_block_dot_equals_decoded_times_q8(oracle, qtype):
    rng = np.random.default_rng(60 + qtype)
    values, nbytes = qb.SHAPE[qtype]
    ncols = 512
    row = qb.random_blocks(rng, qtype, ncols // values)
    w = qb.np_dequant(qtype, row).astype(np.float64)
    x = rng.standard_normal((1, ncols)).astype(np.float32)
    xq = oracle.quantize_q8_1(x).reshape(-1, 36)
    dx = xq[:, 0:2].copy().view(np.float16).astype(np.float64).reshape(-1)
    qx = xq[:, 4:].view(np.int8).astype(np.float64)
    for kb in range(ncols // 32):
        got = float(oracle.lib.fnx_o_vec_dot_type(qtype, ol.ptr(row), kb, ol.ptr(np.ascontiguousarray(xq[kb]))))
        want = float((w[32 * kb:32 * kb + 32] * (dx[kb] * qx[kb])).sum())
        scale = float(np.abs(w[32 * kb:32 * kb + 32]).max() * dx[kb] * 127 * 32)
        # Q4_0 takes its - 8 offset through the block's sum field: the sum of the real activations, rounded to f16
        tol = 2e-3 if qtype in (qb.Q4_0, qb.Q5_1) else 2e-6   # (Q5_1's m likewise multiplies the sum field)
        assert abs(got - want) <= tol * scale, (kb, got, want)

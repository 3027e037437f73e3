"""Parity of the prompt path (prefill routing, matrix-core expert products, the chunk layer) with the CPU oracle,
through the C ABI.

Bar: bit-exact for picks, counts, job bases and job lists (integers), and for f32 -> f16 conversion; relative L2 <= 1e-3
for the matrix-core products (f16 operands identical to the oracle's, only the fp32 summation order differs: ~1e-6
measured); SwiGLU f16 codes within one step in a small share of places (device expf).
"""
import numpy as np
import pytest

import fnx_gpu
from fnx_gpu import random_iq3s

pytestmark = pytest.mark.gpu

REL_L2 = 1e-3
PF = 64


def rel_l2(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return fnx_gpu.Dev()


def zipf_logits(rng, Cn, nexp, s=1.1, scale=3.0):
    """router logits whose picks follow a Zipf popularity over a random permutation of the experts"""
    pop = 1.0 / np.arange(1, nexp + 1) ** s
    bias = np.log(pop / pop.sum())[rng.permutation(nexp)]
    lg = rng.standard_normal((Cn, nexp + 1)).astype(np.float32) * scale
    lg[:, :nexp] += bias.astype(np.float32) * 2
    return lg


@pytest.mark.parametrize("Cn,nexp,topk,zipf", [(512, 512, 10, True), (512, 512, 10, False), (70, 8, 2, False), (1, 64, 4, False),
                                              (300, 1000, 8, True)])
def test_pf_route_bit_exact(dev, oracle, Cn, nexp, topk, zipf):
    print(f"case pf_route C={Cn} nexp={nexp} topk={topk} zipf={zipf}", flush=True)
    rng = np.random.default_rng(700 + Cn + nexp)
    logits = zipf_logits(rng, Cn, nexp) if zipf else rng.standard_normal((Cn, nexp + 1)).astype(np.float32)
    if Cn > 2:
        logits[2, :topk + 3] = logits[2].max() + 1.0   # a run of ties: the lower indexes win
    r = dev.pf_route(logits, nexp, topk)
    topi, topw = oracle.topk_logits(logits, nexp, topk)
    assert np.array_equal(r["topi"], topi)
    assert np.allclose(r["topw"], topw, rtol=2e-6, atol=0)
    gu, dn, cnt = oracle.pf_jobs(topi, nexp, PF)
    assert np.array_equal(r["cnt"], cnt)
    assert r["njobs"] == len(gu)
    assert np.array_equal(r["jbase"], np.concatenate([[0], np.cumsum((cnt + PF - 1) // PF)[:-1]]))
    for got, want in ((r["gu"], gu), (r["dn"], dn)):
        assert np.array_equal(got[:, :2], want[:, :2])
        for g, w in zip(got, want):
            n = w[1]
            assert np.array_equal(g[2:2 + n], w[2:2 + n]) and np.array_equal(g[2 + PF:2 + PF + n], w[2 + PF:2 + PF + n])


def test_pf_route_with_fewer_finite_logits_than_picks(dev, oracle):
    from test_oracle_routing import scarce_logits
    Cn, nexp, topk = 70, 512, 10
    print(f"case pf_route scarce C={Cn} nexp={nexp} topk={topk}", flush=True)
    logits = scarce_logits(np.random.default_rng(705), Cn, nexp)
    r = dev.pf_route(logits, nexp, topk)
    topi, topw = oracle.topk_logits(logits, nexp, topk)
    assert np.array_equal(r["topi"], topi)
    assert all(len(set(row.tolist())) == topk for row in r["topi"])
    assert np.all(np.isfinite(r["topw"])) and np.allclose(r["topw"], topw, rtol=2e-6, atol=0)
    gu, dn, cnt = oracle.pf_jobs(topi, nexp, PF)
    assert np.array_equal(r["cnt"], cnt) and r["njobs"] == len(gu)


def test_f32_f16_bit_exact(dev, oracle):
    rng = np.random.default_rng(710)
    x = (rng.standard_normal((33, 257)) * 10.0 ** rng.integers(-8, 4, (33, 257))).astype(np.float32)
    assert np.array_equal(dev.f32_f16(x).view(np.uint16), oracle.f32_f16(x).view(np.uint16))


def test_swiglu_h16(dev, oracle):
    rng = np.random.default_rng(711)
    gu = (rng.standard_normal((50, 1024)) * 3).astype(np.float32)
    got, want = dev.swiglu_h16(gu, 512).view(np.uint16).astype(np.int32), oracle.swiglu_h16(gu, 512).view(np.uint16).astype(np.int32)
    diff = np.abs(got - want)
    assert diff.max() <= 1 and np.count_nonzero(diff) <= 1e-3 * diff.size


def h16_close(a, b):
    """two kernels' h = f16(silu(gate) * up) from the same f16 operands added up in different orders: nearly every value the
    same f16, the rest a rounding step apart"""
    differ = int((a.view(np.uint16) != b.view(np.uint16)).sum())
    print(f"{differ} of {a.size} f16 values of h differ", flush=True)
    assert differ <= a.size // 100 and rel_l2(a.astype(np.float32), b.astype(np.float32)) <= 1e-4


def make_jobs(rng, nexp, rows_avail, sizes):
    jobs = np.zeros((len(sizes), 2 + 2 * PF), dtype=np.int32)
    at = 0
    for j, n in enumerate(sizes):
        jobs[j, 0], jobs[j, 1] = rng.integers(0, nexp), n
        jobs[j, 2:2 + n] = rng.choice(rows_avail, size=n, replace=False)
        jobs[j, 2 + PF:2 + PF + n] = np.arange(at, at + n)
        at += n
    return jobs, at


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("nrows,ncols,down", [(1024, 2048, False), (2048, 512, True), (64, 256, False), (512, 1024, True)])
def test_moe_mma_matches_oracle(dev, oracle, nrows, ncols, down, packed):
    print(f"case moe_mma nrows={nrows} ncols={ncols} down={down} packed={packed}", flush=True)
    if packed and (nrows * ncols) % 2048:
        pytest.skip("unit64 takes whole units of 2048 weights")
    rng = np.random.default_rng(720 + nrows + ncols)
    nexp = 3
    stride = nrows * ncols // 256 * 110
    w = random_iq3s(rng, nexp * nrows * ncols // 256, dmax=2e-2)
    x16 = rng.standard_normal((200, ncols)).astype(np.float16)
    jobs, total = make_jobs(rng, nexp, 200, [64, 1, 17, 16, 33, 48, 5])
    want = oracle.moe_mma(w, stride, nrows, ncols, jobs, PF, x16, total)
    # the arrays hold more jobs than the count says: the rest must not run (their entries are zero: n = 0)
    got = dev.moe_mma(w, stride, nrows, ncols, jobs, x16, total, packed=packed, down=down, cap=len(jobs) + 5)
    assert rel_l2(got, want) <= REL_L2
    assert rel_l2(got, want) <= 1e-5, "f16 operands are the oracle's: only the summation order may differ"


@pytest.mark.parametrize("nrows,nexp,sizes", [(2048, 40, [64, 1, 17, 0, 16, 33, 48, 5, 64, 64, 2, 0, 31, 64, 49, 15] * 6), (64, 3, [64, 1, 17, 16, 33, 48, 5]),
                                              (32, 2, [3]), (2048, 2, [64])])
def test_moe_mma_wave_form_tile16_rows_of_512(dev, oracle, nrows, nexp, sizes):
    # the down projection over tile16 matrices of 512 columns (k_moe_mma_wave16): blocks that end inside a job and blocks
    # that hold several, jobs without tokens, fewer items than blocks
    print(f"case moe_mma wave form nrows={nrows} nexp={nexp} jobs={len(sizes)}", flush=True)
    ncols = 512
    rng = np.random.default_rng(733 + nrows + len(sizes))
    stride = nrows * ncols // 256 * 110
    w = random_iq3s(rng, nexp * nrows * ncols // 256, dmax=2e-2)
    rows = max(200, sum(sizes))
    x16 = rng.standard_normal((rows, ncols)).astype(np.float16)
    jobs, total = make_jobs(rng, nexp, rows, sizes)
    got = dev.moe_mma(w, stride, nrows, ncols, jobs, x16, total, packed=True, down=True, cap=len(jobs) + 5, tile16=True)
    other = dev.moe_mma(w, stride, nrows, ncols, jobs, x16, total, packed=True, down=True, cap=len(jobs) + 5)   # the wave-a-task kernel over unit64
    assert rel_l2(got, other) <= 1e-6, "the same f16 products: only the summation order differs"
    assert np.array_equal(got == 0, other == 0)   # (rows no job writes stay as they were)
    if len(sizes) <= 8:
        want = oracle.moe_mma(w, stride, nrows, ncols, jobs, PF, x16, total)
        assert rel_l2(got, want) <= 1e-5, "f16 operands are the oracle's: only the summation order may differ"


@pytest.mark.parametrize("ffs,ncols,nexp,sizes", [(512, 2048, 24, [64, 1, 17, 0, 16, 33, 48, 5, 64, 64, 2, 0, 31, 64, 49, 15] * 3), (128, 512, 3, [64, 1, 17, 16, 33, 48, 5]),
                                                  (256, 1024, 2, [3]), (640, 2048, 2, [64, 9]), (128, 2560, 2, [5, 64, 20, 16])])
def test_moe_gate_up_h16_one_launch_equals_two(dev, oracle, ffs, ncols, nexp, sizes):
    # h = silu(gate) * up straight from the matrix-core launch (the wave form over tile16) against fnx_moe_gate_up_mma over
    # the unit64 copy followed by fnx_swiglu_h16, whatever the mix of job sizes, with rows no job writes left alone
    # (640: a job's last unit is short of pairs; 2560 columns: five activation tiles a row, so small jobs go as heavy units)
    tile16 = True
    print(f"case moe_gate_up_h16 ffs={ffs} ncols={ncols} nexp={nexp} jobs={len(sizes)}", flush=True)
    nrows = 2 * ffs
    rng = np.random.default_rng(741 + ffs + len(sizes))
    stride = nrows * ncols // 256 * 110
    w = random_iq3s(rng, nexp * nrows * ncols // 256, dmax=2e-2)
    rows = max(200, sum(sizes))
    x16 = rng.standard_normal((rows, ncols)).astype(np.float16)
    jobs, total = make_jobs(rng, nexp, rows, sizes)
    one, two = dev.moe_mma(w, stride, nrows, ncols, jobs, x16, total + 3, packed=True, cap=len(jobs) + 5, tile16=tile16, h16=True)
    assert np.all(np.isfinite(two.astype(np.float32)))
    # the same f16 operands on both sides; the two kernels add a row's products in different orders, which now and then moves
    # an f16 value of h by one step
    h16_close(one, two)
    assert np.any(one[:total] != 0) and not np.any(one[total:])
    if len(sizes) <= 8:   # against the oracle: its products, its SwiGLU
        gu = oracle.moe_mma(w, stride, nrows, ncols, jobs, PF, x16, total + 3)
        want = oracle.swiglu_h16(gu, ffs)
        assert rel_l2(one.astype(np.float32), want.astype(np.float32)) <= 1e-3


def split_in_16s(jobs):
    """jobs of up to 64 rows as the jobs of up to 16 rows they consist of (the oracle's mmvq takes those)"""
    out = []
    for jb in jobs:
        n = int(jb[1])
        for t0 in range(0, n, 16):
            k = min(16, n - t0)
            j = np.zeros(1, dtype=fnx_gpu.JOB_DTYPE)
            j["w"], j["n"] = jb[0], k
            j["y"][0, :k], j["out"][0, :k] = jb[2 + t0:2 + t0 + k], jb[2 + PF + t0:2 + PF + t0 + k]
            out.append(j)
    return np.concatenate(out) if out else np.zeros(0, dtype=fnx_gpu.JOB_DTYPE)


@pytest.mark.parametrize("nrows,ncols,nexp,sizes", [(1024, 2048, 24, [64, 1, 17, 0, 16, 33, 48, 5, 64, 64, 2, 0, 31, 64, 49, 15] * 3), (64, 512, 3, [64, 1, 17, 16, 33, 48, 5]),
                                                  (32, 1024, 2, [3]), (2048, 512, 2, [64, 9, 0, 0, 40])])
def test_moe_big_jobs_over_q8_1_match_the_oracle(dev, oracle, nrows, ncols, nexp, sizes):
    """kernels.hpp:324-325: the prompt path's jobs with mmvq's terms. gate|up form: q8_1 rows in, the oracle's mmvq over the same
    jobs cut into sixteens; down form (where the matrix's columns allow rows [gate | up]): h = silu(gate) * up quantised on
    the way, against the oracle's SwiGLU -> q8_1 -> mmvq. The integer sums are exact; a row's sub-block terms are added in
    another order than the oracle's."""
    print(f"case moe_big nrows={nrows} ncols={ncols} nexp={nexp} jobs={len(sizes)}", flush=True)
    rng = np.random.default_rng(771 + nrows + len(sizes))
    stride = nrows * ncols // 256 * 110
    w = random_iq3s(rng, nexp * nrows * ncols // 256, dmax=2e-2)
    rows = max(200, sum(sizes))
    jobs, total = make_jobs(rng, nexp, rows, sizes)
    small = split_in_16s(jobs)
    x = rng.standard_normal((rows, ncols)).astype(np.float32)
    xq = oracle.quantize_q8_1(x)
    want = oracle.mmvq(w, stride, nrows, ncols, small, xq, total + 3)
    got = dev.moe_big(w, stride, nrows, ncols, jobs, xq, total + 3, cap=len(jobs) + 5)
    assert rel_l2(got, want) <= 1e-5
    assert np.any(got[:total] != 0) and not np.any(got[total:])
    # the down form: the same matrix read as rows of ncols = ffs, fed rows [gate | up]
    gu = (rng.standard_normal((rows, 2 * ncols)) * 2).astype(np.float32)
    hq = oracle.swiglu_stacked_q8_1(gu, ncols)
    want = oracle.mmvq(w, stride, nrows, ncols, small, hq, total + 3)
    got = dev.moe_big(w, stride, nrows, ncols, jobs, gu, total + 3, down=True, cap=len(jobs) + 5)
    assert rel_l2(got, want) <= 1e-5
    assert not np.any(got[total:])


def test_moe_mma_weights_equal_the_oracles_f16(dev, oracle):
    # x = unit vectors: the product returns single weights, so every dequantised f16 value is checked bit for bit,
    # subnormal ones included (tiny d)
    rng = np.random.default_rng(730)
    nrows, ncols = 32, 256
    for dmax in (2e-2, 3e-6):
        w = random_iq3s(rng, nrows * ncols // 256, dmax=dmax)
        want = oracle.iq3s_dequant_f16(w).reshape(nrows, ncols)
        x16 = np.eye(ncols, dtype=np.float16)
        jobs = np.zeros((4, 2 + 2 * PF), dtype=np.int32)
        for j in range(4):
            jobs[j, 1] = 64
            jobs[j, 2:2 + 64] = np.arange(64 * j, 64 * j + 64)
            jobs[j, 2 + PF:] = np.arange(64 * j, 64 * j + 64)
        for packed in (False, True):
            got = dev.moe_mma(w, 0, nrows, ncols, jobs, x16, ncols, packed=packed)
            assert np.array_equal(got.T.astype(np.float16).view(np.uint16), want.view(np.uint16))
            assert np.array_equal(got.T, want.astype(np.float32))


@pytest.mark.parametrize("n,ff,nexp,topk,Cn", [(2048, 512, 32, 4, 100), (2048, 512, 512, 10, 64), (256, 256, 8, 2, 70)])
def test_prefill_layer_matches_oracle(dev, oracle, n, ff, nexp, topk, Cn):
    print(f"case prefill_layer n={n} ff={ff} nexp={nexp} topk={topk} C={Cn}", flush=True)
    rng = np.random.default_rng(740 + nexp + Cn)   # d small enough that h = silu(g) u stays inside f16's range
    nb = lambda rows, cols: rows * cols // 256
    gu = random_iq3s(rng, nexp * nb(2 * ff, n), dmax=1e-3)
    down = random_iq3s(rng, nexp * nb(n, ff), dmax=1e-3)
    sh_gu, sh_down = random_iq3s(rng, nb(2 * ff, n), dmax=1e-3), random_iq3s(rng, nb(n, ff), dmax=1e-3)
    router = (rng.standard_normal((nexp + 1, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((Cn, n)).astype(np.float32)
    want = oracle.moe_prefill_layer(n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x)
    packed = (2 * ff * n) % 2048 == 0 and (n * ff) % 2048 == 0
    L = fnx_gpu.PfLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, Cn, packed=packed)
    for rep in range(2):   # a second chunk through the same workspace
        r = L.run(x)
        assert np.array_equal(r["logits"].view(np.uint32), want["logits"].view(np.uint32))
        assert np.array_equal(r["topi"], want["topi"])
        assert int(r["njobs"][0]) == want["njobs"] and int(r["njobs"][1]) == (Cn + PF - 1) // PF
        assert np.all(np.isfinite(want["out"]))
        assert rel_l2(r["out"], want["out"]) <= REL_L2


@pytest.mark.parametrize("n,ff,nexp,topk,Cn", [(2048, 512, 48, 10, 300), (1024, 256, 8, 2, 70)])
def test_prefill_layer_tile16_equals_unit64(dev, oracle, n, ff, nexp, topk, Cn):
    """the gate|up matrices (and the down matrices, where ff comes in 512s) in the prompt path's own layout: the same f16
    weights and activations as the unit64 layout's kernel, whose tasks add a row's products up in another order, so h and the
    chunk's result agree to float rounding (and with the oracle's within the bar either way)"""
    print(f"case prefill_layer tile16 n={n} ff={ff} nexp={nexp} topk={topk} C={Cn}", flush=True)
    rng = np.random.default_rng(760 + nexp)
    nb = lambda rows, cols: rows * cols // 256
    gu = random_iq3s(rng, nexp * nb(2 * ff, n), dmax=1e-3)
    down = random_iq3s(rng, nexp * nb(n, ff), dmax=1e-3)
    sh_gu, sh_down = random_iq3s(rng, nb(2 * ff, n), dmax=1e-3), random_iq3s(rng, nb(n, ff), dmax=1e-3)
    router = (rng.standard_normal((nexp + 1, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((Cn, n)).astype(np.float32)
    a = fnx_gpu.PfLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, Cn, packed=True).run(x)
    b = fnx_gpu.PfLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, Cn, packed=True, tile16=True).run(x)
    assert np.array_equal(a["topi"], b["topi"])
    h16_close(a["h16"], b["h16"])
    assert rel_l2(b["out"], a["out"]) <= 1e-5
    want = oracle.moe_prefill_layer(n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x)
    assert rel_l2(b["out"], want["out"]) <= REL_L2


@pytest.mark.parametrize("tile16,Cn", [(False, 8192), (True, 8192), (True, 2048)])
def test_prefill_layer_large_chunk_equals_small_chunks(dev, tile16, Cn):
    """A size-independent property at a size the oracle does not reach: a row's result does not depend on what else is in
    its chunk, so 8,192 rows in one call (more tasks than one pass of a block's task list holds, every kernel form's loop
    over list passes, a thousand jobs and more split over the wave form's blocks) must equal the same rows in 16 calls of
    512, bit for bit, in either layout. (2,048 rows: a few hundred jobs, ranked, their heavy units several to a block.)"""
    n, ff, nexp, topk, small = 2048, 512, 64, 10, 512
    print(f"case prefill_layer large n={n} ff={ff} nexp={nexp} topk={topk} C={Cn} tile16={tile16}", flush=True)
    rng = np.random.default_rng(777)
    nb = lambda rows, cols: rows * cols // 256
    gu = random_iq3s(rng, nexp * nb(2 * ff, n), dmax=1e-3)
    down = random_iq3s(rng, nexp * nb(n, ff), dmax=1e-3)
    sh_gu, sh_down = random_iq3s(rng, nb(2 * ff, n), dmax=1e-3), random_iq3s(rng, nb(n, ff), dmax=1e-3)
    router = (rng.standard_normal((nexp + 1, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((Cn, n)).astype(np.float32)
    big = fnx_gpu.PfLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, Cn, packed=True, tile16=tile16).run(x)["out"]
    L = fnx_gpu.PfLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, small, packed=True, tile16=tile16)
    assert np.all(np.isfinite(big))
    for c0 in range(0, Cn, small):
        part = L.run(x[c0:c0 + small])["out"]
        assert int(np.count_nonzero(part.view(np.uint32) != big[c0:c0 + small].view(np.uint32))) == 0, f"rows {c0}.."


def test_prefill_layer_two_chunks_in_flight(dev):
    """A layer's chunks are independent, and a call's state is all in its workspace: chunks dealt to two streams with a
    workspace each must leave the bits that the same chunks leave one after the other on one stream."""
    import ctypes as C
    n, ff, nexp, topk, Cn, chunks = 2048, 512, 64, 10, 512, 6
    print(f"case prefill_layer two streams n={n} ff={ff} nexp={nexp} topk={topk} C={Cn}", flush=True)
    rng = np.random.default_rng(778)
    nb = lambda rows, cols: rows * cols // 256
    gu = random_iq3s(rng, nexp * nb(2 * ff, n), dmax=1e-3)
    down = random_iq3s(rng, nexp * nb(n, ff), dmax=1e-3)
    sh_gu, sh_down = random_iq3s(rng, nb(2 * ff, n), dmax=1e-3), random_iq3s(rng, nb(n, ff), dmax=1e-3)
    router = (rng.standard_normal((nexp + 1, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((chunks, Cn, n)).astype(np.float32)
    A = fnx_gpu.PfLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, Cn, packed=True, tile16=True)
    B = fnx_gpu.PfLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, Cn, packed=True, tile16=True)
    want = [A.run(x[c])["out"] for c in range(chunks)]
    t = dev.torch
    dx = dev.up(x)
    outs = dev.zeros((chunks, Cn, n), t.float32)
    streams = [t.cuda.Stream(), t.cuda.Stream()]
    t.cuda.synchronize()
    for rep in range(3):
        outs.zero_()
        t.cuda.synchronize()
        for c in range(chunks):
            L, s = ((A, streams[0]), (B, streams[1]))[c & 1]
            dev.ok(dev.lib.fnx_moe_prefill_layer(C.byref(L.L), dx[c].data_ptr(), Cn, outs[c].data_ptr(), C.byref(L.ws), s.cuda_stream))
        t.cuda.synchronize()
        got = outs.cpu().numpy()
        for c in range(chunks):
            assert int(np.count_nonzero(got[c].view(np.uint32) != want[c].view(np.uint32))) == 0, f"round {rep}, chunk {c}"

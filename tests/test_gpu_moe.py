"""Parity of the MoE verify layer (benchmark config 2) with the CPU oracle: op by op and as one call."""
import ctypes as C
import os
import subprocess
import sys

import numpy as np
import pytest

import fnx_gpu
from fnx_gpu import random_iq3s

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return fnx_gpu.Dev()


def make_layer(rng, n, ff, nexp, scale=1.0):
    router = (rng.standard_normal((nexp + 1, n)) * 0.02 * scale).astype(np.float32)
    gu = random_iq3s(rng, nexp * 2 * ff * n // 256)
    down = random_iq3s(rng, nexp * n * ff // 256)
    sh_gu = random_iq3s(rng, 2 * ff * n // 256)
    sh_down = random_iq3s(rng, n * ff // 256)
    return router, gu, down, sh_gu, sh_down


def check_jobs(got, want):
    for g, w in zip(got, want):
        k = int(w["n"])
        assert int(g["w"]) == int(w["w"]) and int(g["n"]) == k
        assert np.array_equal(g["y"][:k], w["y"][:k]) and np.array_equal(g["out"][:k], w["out"][:k])


def check_layer(dev, oracle, n, ff, nexp, topk, T, seed, packed=False):
    """packed: the unit64 layout (eligible shapes then run as the one-launch window)"""
    print(f"case moe layer n={n} ff={ff} nexp={nexp} topk={topk} T={T} seed={seed} packed={packed}", flush=True)
    rng = np.random.default_rng(seed)
    router, gu, down, sh_gu, sh_down = make_layer(rng, n, ff, nexp)
    x = rng.standard_normal((T, n)).astype(np.float32)
    want = oracle.moe_verify_layer(n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x)
    layer = fnx_gpu.MoeLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, packed=packed)
    layer.raw = (gu, down, sh_gu, sh_down)
    got = layer.run(x)
    assert not got["sync"].any(), "no block gave up a wait, and the window put its arrival counters back to zero"
    assert np.array_equal(got["logits"].view(np.uint32), want["logits"].view(np.uint32)), "router logits bit-exact"
    assert np.array_equal(got["topi"], want["topi"]), "routing picks bit-exact"
    assert got["njobs"] == want["njobs"]
    assert np.array_equal(got["topw"].view(np.uint32), want["topw"].view(np.uint32)), "routing weights bit-exact (one exp on both sides)"
    gu_jobs, dn_jobs = oracle.jobs(want["topi"])
    check_jobs(got["jobs_gu"][:got["njobs"]], gu_jobs)
    check_jobs(got["jobs_dn"][:got["njobs"]], dn_jobs)
    # One exp on both sides (include/fnx_expf.h) and the row sums in the reference's butterfly order: the q8_1 codes of h are
    # the oracle's, and so is every bit of the layer's output, in either layout
    assert np.array_equal(got["out"].view(np.uint32), want["out"].view(np.uint32)), rel_l2(got["out"], want["out"])
    return got, want, layer, x


@pytest.mark.parametrize("packed", [False, True])
def test_moe_verify_layer_config2(dev, oracle, packed):
    # hidden 2048, 512 experts, top-10, SwiGLU experts 2048 -> 512 -> 2048, one shared expert, T = 16
    got, want, layer, x = check_layer(dev, oracle, 2048, 512, 512, 10, 16, 900, packed)
    # a second window on the same layer and workspace, fewer rows
    rng = np.random.default_rng(901)
    x2 = rng.standard_normal((5, 2048)).astype(np.float32)
    router = layer.router.cpu().numpy()
    want2 = oracle.moe_verify_layer(2048, 512, 512, 10, router, *layer.raw, x2)
    got2 = layer.run(x2)
    assert np.array_equal(got2["topi"], want2["topi"]) and got2["njobs"] == want2["njobs"]
    assert np.array_equal(got2["out"].view(np.uint32), want2["out"].view(np.uint32))


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("n,ff,nexp,topk,T", [(2048, 512, 64, 10, 1), (1024, 256, 32, 4, 16), (2048, 1024, 16, 2, 3), (512, 512, 16, 8, 7),
                                              (2048, 256, 40, 6, 9), (2048, 512, 1000, 10, 16), (2048, 512, 12, 10, 16),
                                              # windows of few rows: a block has four or eight units and deals the row's trips over its waves
                                              (2048, 512, 64, 10, 2), (2048, 512, 128, 10, 4), (2048, 512, 512, 10, 3)])
def test_moe_verify_layer_shapes(dev, oracle, n, ff, nexp, topk, T, packed):
    # with unit64 weights the shapes of hidden 2048 run as the one-launch window, the others operator by operator
    check_layer(dev, oracle, n, ff, nexp, topk, T, 910 + T, packed)


@pytest.mark.parametrize("packed", [False, True])
def test_moe_verify_layer_with_experts_from_pointer_tables(dev, oracle, packed):
    """fnx_dw.ep: an expert's matrix by a table of device pointers instead of base + e * stride (an engine whose experts
    sit in allocations of their own). The tables here list the experts in a shuffled memory order and the bases are null,
    so only a launch that goes by the tables can give the oracle's bits."""
    import torch
    n, ff, nexp, topk, T = 2048, 512, 48, 10, 16
    got, want, layer, x = check_layer(dev, oracle, n, ff, nexp, topk, T, 930, packed)
    rng = np.random.default_rng(931)
    perm = rng.permutation(nexp)   # expert e's matrices lie at place perm[e]
    tables = []
    for w, stride in ((layer.gu, layer.gu_stride), (layer.down, layer.down_stride)):
        moved = torch.empty_like(w)
        src = w.view(nexp, stride)
        moved.view(nexp, stride)[torch.as_tensor(perm, device=w.device)] = src
        table = torch.as_tensor(moved.data_ptr() + perm.astype(np.int64) * stride, dtype=torch.int64, device=w.device)
        tables.append((moved, table))
    layer.L.gu.p = layer.L.down.p = None
    layer.L.gu.ep, layer.L.down.ep = tables[0][1].data_ptr(), tables[1][1].data_ptr()
    got2 = layer.run(x)
    assert not got2["sync"].any()
    assert np.array_equal(got2["topi"], want["topi"])
    assert np.array_equal(got2["out"].view(np.uint32), want["out"].view(np.uint32)), rel_l2(got2["out"], want["out"])


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("n,ff,nexp,topk,T", [(2048, 512, 512, 10, 16), (2048, 256, 40, 6, 3)])
def test_moe_verify_layer_with_a_bf16_router(dev, oracle, n, ff, nexp, topk, T, packed):
    """fnx_moe_layer.router_bf16: the router's rows as bf16 (the upper halves of f32 values), multiplied as the f32 values
    they stand for - so the oracle over those f32 values gives the bits."""
    import torch
    rng = np.random.default_rng(940 + T)
    router, gu, down, sh_gu, sh_down = make_layer(rng, n, ff, nexp)
    bits = (router.view(np.uint32) >> 16).astype(np.uint16)             # truncated to bf16
    router_as_f32 = (bits.astype(np.uint32) << 16).view(np.float32)
    x = rng.standard_normal((T, n)).astype(np.float32)
    want = oracle.moe_verify_layer(n, ff, nexp, topk, router_as_f32, gu, down, sh_gu, sh_down, x)
    layer = fnx_gpu.MoeLayerDev(dev, n, ff, nexp, topk, router_as_f32, gu, down, sh_gu, sh_down, packed=packed)
    rb = torch.from_numpy(bits.view(np.int16).copy()).to("cuda")
    layer.L.router, layer.L.router_bf16 = rb.data_ptr(), 1
    got = layer.run(x)
    assert not got["sync"].any()
    assert np.array_equal(got["logits"].view(np.uint32), want["logits"].view(np.uint32)), "router logits bit-exact"
    assert np.array_equal(got["topi"], want["topi"])
    assert np.array_equal(got["out"].view(np.uint32), want["out"].view(np.uint32)), rel_l2(got["out"], want["out"])


def q8_split(oracle, rng, rows, cols, scale):
    import oracle_lib as ol
    w = (rng.standard_normal((rows, cols)) * scale).astype(np.float32)
    q, d = np.zeros((rows, cols), dtype=np.int8), np.zeros((rows, cols // 32), dtype=np.uint16)
    oracle.lib.fnx_o_quantize_q8_0_split(ol.ptr(w), rows, cols, ol.ptr(q), ol.ptr(d))
    return q, d


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("n,ff,nexp,topk,T", [(2048, 512, 512, 10, 16), (2048, 512, 64, 1, 3), (2048, 256, 24, 4, 7)])
def test_moe_verify_layer_with_a_q8_0_shared_expert(dev, oracle, n, ff, nexp, topk, T, packed):
    """the reference's own form of the shared expert (engine.cu:1600-1604: split Q8_0 through q8s_gemv ->
    swiglu_stacked_q8_1 -> q8s_gemv) beside IQ3_S routed experts: with unit64 experts inside the one-launch window,
    with raw blocks operator by operator"""
    print(f"case moe layer q8_0 shared n={n} ff={ff} nexp={nexp} topk={topk} T={T} packed={packed}", flush=True)
    rng = np.random.default_rng(940 + T)
    router, gu, down, sh_gu, sh_down = make_layer(rng, n, ff, nexp)
    sh_q8 = (q8_split(oracle, rng, 2 * ff, n, 0.02), q8_split(oracle, rng, n, ff, 0.02))
    layer = fnx_gpu.MoeLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, packed=packed, sh_q8=sh_q8)
    for rows in (T, max(1, T // 2)):   # a second, shorter window on the same workspace
        x = rng.standard_normal((rows, n)).astype(np.float32)
        want = oracle.moe_verify_layer(n, ff, nexp, topk, router, gu, down, None, None, x, sh_q8=sh_q8)
        with_iq3s = oracle.moe_verify_layer(n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x)
        assert rel_l2(want["out"], with_iq3s["out"]) > 1e-2, "the two shared experts differ, so the test tells them apart"
        got = layer.run(x)
        assert np.array_equal(got["logits"].view(np.uint32), want["logits"].view(np.uint32))
        assert np.array_equal(got["topi"], want["topi"]) and got["njobs"] == want["njobs"]
        err = rel_l2(got["out"], want["out"])
        print("rel l2", err, flush=True)
        assert err <= 1e-3


@pytest.mark.parametrize("packed", [False, True])
def test_two_windows_on_two_streams(dev, oracle, packed):
    """two layers, each with a workspace of its own, their windows enqueued on two streams with nothing between them: the
    results are the single-stream ones. With unit64 weights a window touches only its workspace; operator by operator
    the pairs' q8_1 rows go through the library's one buffer per device, and the library puts the calls in order."""
    import ctypes as C
    t = dev.torch
    n, ff, nexp, topk, T = 2048, 512, 48, 10, 16
    rng = np.random.default_rng(950)
    layers, xs, want = [], [], []
    for i in range(2):
        router, gu, down, sh_gu, sh_down = make_layer(rng, n, ff, nexp)
        layers.append(fnx_gpu.MoeLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, packed=packed))
        xs.append([rng.standard_normal((T, n)).astype(np.float32) for _ in range(6)])
        want.append([layers[i].run(x)["out"] for x in xs[i]])   # one at a time, each waited for
    streams = [t.cuda.Stream(), t.cuda.Stream()]
    dxs = [[dev.up(x) for x in xs[i]] for i in range(2)]
    outs = [[dev.zeros((T, n), t.float32) for _ in xs[i]] for i in range(2)]
    dev.sync()
    print(f"case two streams packed={packed}", flush=True)
    for j in range(6):
        for i in range(2):
            with t.cuda.stream(streams[i]):
                dev.ok(dev.lib.fnx_moe_verify_layer(C.byref(layers[i].L), dxs[i][j].data_ptr(), T, outs[i][j].data_ptr(), C.byref(layers[i].ws), dev.st()))
    for s_ in streams:
        s_.synchronize()
    for i in range(2):
        for j in range(6):
            assert np.array_equal(outs[i][j].cpu().numpy().view(np.uint32), want[i][j].view(np.uint32)), (i, j)


def test_moe_verify_layer_repeated_windows(dev, oracle):
    # many windows back to back on one layer and workspace, varying T
    rng = np.random.default_rng(930)
    n, ff, nexp, topk = 2048, 512, 64, 10
    router, gu, down, sh_gu, sh_down = make_layer(rng, n, ff, nexp)
    layer = fnx_gpu.MoeLayerDev(dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, packed=True)
    for i, T in enumerate([16, 1, 7, 16, 3, 12]):
        print(f"case repeated window {i} T={T}", flush=True)
        x = rng.standard_normal((T, n)).astype(np.float32)
        want = oracle.moe_verify_layer(n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x)
        got = layer.run(x)
        assert np.array_equal(got["topi"], want["topi"]) and got["njobs"] == want["njobs"]
        assert np.array_equal(got["out"].view(np.uint32), want["out"].view(np.uint32))


def test_moe_ops_one_by_one_equal_the_fused_call(dev, oracle):
    # the reference's call sequence (engine.cu:1569-1757): quantize, router_route, gate|up, down, shared expert, combine
    n, ff, nexp, topk, T = 2048, 512, 64, 10, 16
    got, want, layer, x = check_layer(dev, oracle, n, ff, nexp, topk, T, 920)
    t, lib, pkg = dev.torch, dev.lib, dev.pkg
    P = T * topk
    dx = dev.up(x)
    xq = dev.zeros(T * (n // 32) * 36, t.uint8)
    logits, topi, topw = dev.zeros((T, nexp + 1), t.float32), dev.zeros((T, topk), t.int32), dev.zeros((T, topk), t.float32)
    jgu, jdn, nj = dev.zeros(P * 136, t.uint8), dev.zeros(P * 136, t.uint8), dev.zeros(2, t.int32)
    gu, part, out = dev.zeros((P + T, 2 * ff), t.float32), dev.zeros((P + T, n), t.float32), dev.zeros((T, n), t.float32)
    st = dev.st()
    dev.ok(lib.fnx_quantize_q8_1(dx.data_ptr(), xq.data_ptr(), n, T, st))
    dev.ok(lib.fnx_router_route(layer.router.data_ptr(), 0, dx.data_ptr(), logits.data_ptr(), T, n, nexp, topk, topi.data_ptr(),
                                topw.data_ptr(), jgu.data_ptr(), jdn.data_ptr(), nj.data_ptr(), st))
    dev.ok(lib.fnx_moe_gate_up(C.byref(layer.L.gu), layer.gu_stride, jgu.data_ptr(), nj.data_ptr(), P, xq.data_ptr(), gu.data_ptr(), topk, st))
    dev.ok(lib.fnx_moe_down(C.byref(layer.L.down), layer.down_stride, jdn.data_ptr(), nj.data_ptr(), P, gu.data_ptr(), part.data_ptr(), st))
    # the shared expert as the reference runs it: a dense gate|up over all rows, swiglu to q8_1, a dense down
    sh_job = np.zeros(1, dtype=fnx_gpu.JOB_DTYPE)
    sh_job["n"] = T
    sh_job["y"][0, :T] = np.arange(T)
    sh_job["out"][0, :T] = np.arange(T)
    dj = dev.up(sh_job.view(np.uint8).reshape(-1))
    sh_gu, sh_hq, sh_part = dev.zeros((T, 2 * ff), t.float32), dev.zeros(T * (ff // 32) * 36, t.uint8), dev.zeros((T, n), t.float32)
    dev.ok(lib.fnx_mmvq(C.byref(layer.L.sh_gu), 0, dj.data_ptr(), None, 1, xq.data_ptr(), sh_gu.data_ptr(), 2 * ff, st))
    dev.ok(lib.fnx_swiglu_stacked_q8_1(sh_gu.data_ptr(), sh_hq.data_ptr(), ff, T, st))
    dev.ok(lib.fnx_mmvq(C.byref(layer.L.sh_down), 0, dj.data_ptr(), None, 1, sh_hq.data_ptr(), sh_part.data_ptr(), n, st))
    dev.ok(lib.fnx_moe_combine(part.data_ptr(), topw.data_ptr(), sh_part.data_ptr(), logits[:, nexp:].contiguous().data_ptr(), 1,
                               out.data_ptr(), T, n, topk, st))
    dev.sync()
    # the one-call form is the same arithmetic, the row sums in the same order
    assert np.array_equal(out.cpu().numpy().view(np.uint32), got["out"].view(np.uint32))
    # intermediate checks against the oracle's definitions
    hq_want = oracle.swiglu_stacked_q8_1(sh_gu.cpu().numpy(), ff)
    # q8_1 bytes of h: one exp on both sides, so the same bytes
    assert np.array_equal(sh_hq.cpu().numpy().reshape(-1, 36), hq_want.reshape(-1, 36))
    comb = oracle.moe_combine(part.cpu().numpy()[:P], topw.cpu().numpy(), sh_part.cpu().numpy(), logits.cpu().numpy()[:, nexp])
    assert np.array_equal(out.cpu().numpy().view(np.uint32), comb.view(np.uint32))


def test_a_window_whose_waits_run_out_leaves_and_says_so(dev):
    """the error path of the window's cross-block waits, forced from the host: with no wait budget (a child process, since the
    library reads the budget once) every block still leaves, the launch ends, and the workspace's error word carries
    FNX_ERR_BARRIER - the caller's sign to discard the window's results and zero the sync words before the next one"""
    env = dict(os.environ, FNX_WINDOW_WAIT_TICKS="0")
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "window_timeout_child.py")
    print("case window with no wait budget (child process)", flush=True)
    r = subprocess.run([sys.executable, "-u", child], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stdout + r.stderr
    line = [l for l in r.stdout.splitlines() if l.startswith("window left err=")]
    assert line, r.stdout + r.stderr
    err = int(line[0].split("=")[1])
    assert err & dev.pkg.ERR_BARRIER, "a wait that gives up sets the error bit"

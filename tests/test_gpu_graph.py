"""The operators are asynchronous on the caller's stream, allocate nothing and never synchronise, so a caller can
capture whole windows into a HIP graph (the reference captures its windows, engine_common.cu:993-1007). A captured MoE
window and a captured verify step are replayed several times with fresh inputs and eager work in between, and every
replay is checked against the eager result on the same inputs."""
import ctypes as C

import numpy as np
import pytest

import fnx_gpu
import tiny_decoder as td
from fnx_gpu import random_iq3s

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return fnx_gpu.Dev()


def test_moe_window_in_a_graph(dev):
    torch = dev.torch
    rng = np.random.default_rng(901)
    n, ff, nexp, topk, T = 2048, 512, 64, 6, 16
    nb = lambda rows, cols: rows * cols // 256
    L = fnx_gpu.MoeLayerDev(dev, n, ff, nexp, topk, (rng.standard_normal((nexp + 1, n)) * 0.05).astype(np.float32),
                            random_iq3s(rng, nexp * nb(2 * ff, n)), random_iq3s(rng, nexp * nb(n, ff)), random_iq3s(rng, nb(2 * ff, n)),
                            random_iq3s(rng, nb(n, ff)), T=T, packed=True)
    x_static = torch.zeros((T, n), device="cuda")
    out_static = torch.zeros((T, n), device="cuda")
    xs = [torch.randn((T, n), device="cuda") for _ in range(4)]

    def launch():
        dev.ok(dev.lib.fnx_moe_verify_layer(C.byref(L.L), x_static.data_ptr(), T, out_static.data_ptr(), C.byref(L.ws), dev.st()))

    eager = []
    for x in xs:
        x_static.copy_(x)
        launch()
        torch.cuda.synchronize()
        eager.append(out_static.clone())
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # one warm-up on the capture stream, then the capture
        launch()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch()
    for rep in range(2):
        for x, want in zip(xs, eager):
            x_static.copy_(x)
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_static, want), "a replay reproduces the eager window bit for bit"
            _ = (x * 2).sum().item()   # eager work and a synchronisation between replays


def test_verify_step_in_a_graph(dev, oracle):
    torch = dev.torch
    model = td.TinyDecoder(oracle, seed=21)
    d = fnx_gpu.DecoderDev(dev, model)
    tok_static = torch.zeros(16, dtype=torch.int32, device="cuda")
    windows = [[3, 1, 4, 1, 5, 9, 2, 6], [5, 3, 5, 8, 9, 7, 9, 3], [2, 3, 8, 4, 6, 2, 6, 4]]
    T = 8

    def launch():
        dev.ok(dev.lib.fnx_decoder_verify(C.byref(d.D), tok_static.data_ptr(), T, d.pos.data_ptr(), C.byref(d.ws), dev.st()))

    def run_all(run):
        outs = []
        for i, w in enumerate(windows):
            tok_static[:T] = torch.tensor(w, dtype=torch.int32, device="cuda")
            d.pos.fill_(T * i)
            run()
            torch.cuda.synchronize()
            outs.append((d.b["best_i"][:T].clone(), d.b["logits"][:T].clone()))
        return outs

    eager = run_all(launch)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch()
    replayed = run_all(g.replay)   # the same windows again over the same cache cells: the same results
    for (bi, lg), (bi2, lg2) in zip(eager, replayed):
        assert torch.equal(bi, bi2) and torch.equal(lg, lg2)

"""The window on the library's own workspace (fnx_moe_verify_layer_static): same results as fnx_moe_verify_layer, bit for
bit, on two calls in a row, the second with a smaller window."""
import ctypes as C

import numpy as np
import pytest

import fnx_gpu
from fnx_gpu import random_iq3s

pytestmark = pytest.mark.gpu


def test_static_workspace_window_equals_the_workspace_one():
    import torch
    assert torch.cuda.is_available(), "this test needs the GPU"
    dev = fnx_gpu.Dev()
    rng = np.random.default_rng(4242)
    n, ff, nexp, topk = 2048, 512, 64, 10
    nb = lambda rows, cols: rows * cols // 256
    router = (rng.standard_normal((nexp + 1, n)) * 0.02).astype(np.float32)
    layer = fnx_gpu.MoeLayerDev(dev, n, ff, nexp, topk, router, random_iq3s(rng, nexp * nb(2 * ff, n)), random_iq3s(rng, nexp * nb(n, ff)),
                                random_iq3s(rng, nb(2 * ff, n)), random_iq3s(rng, nb(n, ff)), packed=True)
    for T in (16, 5):   # the second call is smaller and runs on what the first left in the array
        print(f"case static workspace T={T}", flush=True)
        x = rng.standard_normal((T, n)).astype(np.float32)
        want = layer.run(x)["out"]
        dx = dev.up(x)
        out = dev.zeros((T, n), dev.torch.float32)
        dev.ok(dev.lib.fnx_moe_verify_layer_static(C.byref(layer.L), dx.data_ptr(), T, out.data_ptr(), dev.st()))
        dev.sync()
        got = out.cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"T={T}: the two windows differ"
        err = C.c_uint(99)
        dev.ok(dev.lib.fnx_moe_static_status(C.byref(err), dev.st()))
        assert err.value == 0, "no block of the window gave up a wait"
    # shapes beyond the array are refused with a message, before any launch
    raw = fnx_gpu.MoeLayerDev(dev, n, ff, nexp, topk, router, random_iq3s(rng, nexp * nb(2 * ff, n)), random_iq3s(rng, nexp * nb(n, ff)),
                              random_iq3s(rng, nb(2 * ff, n)), random_iq3s(rng, nb(n, ff)), packed=False)
    x = dev.up(rng.standard_normal((4, n)).astype(np.float32))
    out = dev.zeros((4, n), dev.torch.float32)
    assert dev.lib.fnx_moe_verify_layer_static(C.byref(raw.L), x.data_ptr(), 4, out.data_ptr(), dev.st()) != 0
    assert b"one-launch window" in dev.lib.fnx_last_error()
    assert dev.lib.fnx_moe_verify_layer_static(C.byref(layer.L), x.data_ptr(), 17, out.data_ptr(), dev.st()) != 0

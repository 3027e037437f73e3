"""Child process of test_gpu_moe.py's error-path test: a verify window whose cross-block waits are given no time
(FNX_WINDOW_WAIT_TICKS=0 in the environment before the library loads). Every block must still leave: the launch ends, the
workspace's error word carries FNX_ERR_BARRIER, and the process exits normally. Prints one line: "window left err=<word>"."""
import os
import sys

import numpy as np

assert os.environ.get("FNX_WINDOW_WAIT_TICKS") == "0", "run by the test, with the budget set to nothing"
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fnx_gpu  # noqa: E402

dev = fnx_gpu.Dev()
rng = np.random.default_rng(77)
n, ff, nexp, topk, T = 2048, 512, 64, 10, 16
router = (rng.standard_normal((nexp + 1, n)) * 0.02).astype(np.float32)
blocks = lambda k: fnx_gpu.random_iq3s(rng, k)
layer = fnx_gpu.MoeLayerDev(dev, n, ff, nexp, topk, router, blocks(nexp * 2 * ff * n // 256), blocks(nexp * n * ff // 256),
                            blocks(2 * ff * n // 256), blocks(n * ff // 256), packed=True)
print("case window with no wait budget", flush=True)
got = layer.run(rng.standard_normal((T, n)).astype(np.float32))
print(f"window left err={int(got['sync'][0])}", flush=True)

"""A layer's experts from a GGUF file onto the device (fnx_gguf_load_moe_layer: model.cpp:988-989, 1063-1068 without the
other card's half) and through the verify window, against the CPU oracle on the arrays the file was written from.
Bar: router logits, picks and jobs bit-exact, the layer's output within 1e-3 relative L2 (as tests/test_gpu_moe.py)."""
import ctypes as C

import numpy as np
import pytest

import fnx_gpu
import gguf_files as gf

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return fnx_gpu.Dev()


@pytest.mark.parametrize("router_type,ff0,ff1,topk_from_file", [(gf.F32, 0, 512, True), (gf.BF16, 0, 512, False), (gf.F32, 256, 512, False)])
def test_layer_from_gguf_matches_oracle(dev, oracle, tmp_path, router_type, ff0, ff1, topk_from_file):
    t, lib, pkg = dev.torch, dev.lib, dev.pkg
    rng = np.random.default_rng(77)
    n, ff_total, nexp, topk, T, layer = 2048, 512, 24, 10, 16, 7
    ts, a = gf.moe_layer_tensors(rng, layer, n, ff_total, nexp, fnx_gpu.random_iq3s, router_type)
    # the layer's tensors over two shards, other tensors between them
    filler = ("blk.7.attn_norm.weight", gf.F32, [n], rng.standard_normal(n).astype(np.float32).tobytes())
    keys = [gf.kv("general.architecture", gf.STR, "fnxtest"), gf.kv("fnxtest.expert_used_count", gf.U32, topk)]
    first = gf.write(tmp_path / "layer-00001-of-00002.gguf", [filler] + ts[:4], keys=keys)
    gf.write(tmp_path / "layer-00002-of-00002.gguf", ts[4:], keys=[])
    print(f"case gguf layer router={router_type} ff=[{ff0},{ff1}) topk_from_file={topk_from_file}", flush=True)
    g = lib.fnx_gguf_open(first.encode())
    assert g, lib.fnx_last_error()
    z = pkg.MoeBufs()
    dev.ok(lib.fnx_gguf_moe_layer_bytes(g, layer, ff0, ff1, C.byref(z)))
    bufs = [dev.zeros(getattr(z, k + "_bytes"), t.uint8) for k in ("router", "gu", "down", "sh_gu", "sh_down")]
    for k, b in zip(("router", "gu", "down", "sh_gu", "sh_down"), bufs):
        setattr(z, k, b.data_ptr())
    L = pkg.MoeLayer()
    dev.ok(lib.fnx_gguf_load_moe_layer(g, layer, ff0, ff1, 0 if topk_from_file else topk, C.byref(z), C.byref(L), dev.st()))
    dev.sync()
    lib.fnx_gguf_close(g)   # the device copies stand on their own
    ff = ff1 - ff0
    assert (L.n, L.ff, L.nexp, L.topk, L.gu.type, L.gu_stride, L.down_stride) == (n, ff, nexp, topk, pkg.T_IQ3S_UNIT64, 2 * ff * 880, n * ff // 256 * 110)
    # the same slices for the oracle
    gu = gf.slice_rows2(a["gate"], a["up"], n, ff_total, nexp, ff0, ff1)
    down = gf.slice_cols(a["down"], n, ff_total, nexp, ff0, ff1)
    sh_gu = gf.slice_rows2(a["sh_gate"], a["sh_up"], n, ff_total, 1, ff0, ff1)
    sh_down = gf.slice_cols(a["sh_down"], n, ff_total, 1, ff0, ff1)
    router = np.concatenate([a["router"], a["sh_router"]])
    x = rng.standard_normal((T, n)).astype(np.float32)
    want = oracle.moe_verify_layer(n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x)
    # a workspace as MoeLayerDev makes it
    P = T * topk
    w = dict(xq=dev.zeros(T * (n // 32) * 36, t.uint8), logits=dev.zeros((T, nexp + 1), t.float32), topi=dev.zeros((T, topk), t.int32),
             topw=dev.zeros((T, topk), t.float32), jobs_gu=dev.zeros((P + 1) * 136, t.uint8), jobs_dn=dev.zeros((P + 1) * 136, t.uint8),
             njobs=dev.zeros(2, t.int32), gu=dev.zeros((P + T, 2 * ff), t.float32), part=dev.zeros((P + T, n), t.float32),
             sync=dev.zeros(pkg.MOE_SYNC_WORDS, t.int32))
    ws = pkg.MoeWs(*(w[k].data_ptr() for k in ("xq", "logits", "topi", "topw", "jobs_gu", "jobs_dn", "njobs", "gu", "part", "sync")))
    dx, out = dev.up(x), dev.zeros((T, n), t.float32)
    dev.ok(lib.fnx_moe_verify_layer(C.byref(L), dx.data_ptr(), T, out.data_ptr(), C.byref(ws), dev.st()))
    dev.sync()
    assert np.array_equal(w["logits"].cpu().numpy().view(np.uint32), want["logits"].view(np.uint32)), "router logits bit-exact"
    assert np.array_equal(w["topi"].cpu().numpy(), want["topi"]) and int(w["njobs"][0].item()) == want["njobs"]
    assert rel_l2(out.cpu().numpy(), want["out"]) <= 1e-3


def test_layer_with_other_expert_types_from_gguf(dev, oracle, tmp_path):
    """Routed experts in Q4_K, the shared expert in Q8_0 (what a file with K-quant experts holds once its dense tensors
    are Q8_0): loaded as the file has them, the window runs operator by operator; expected = the oracle's operators in
    the reference's order (engine.cu:1569-1757)."""
    import ctypes as C
    import oracle_lib as ol
    import qtype_blocks as qb
    t, lib, pkg = dev.torch, dev.lib, dev.pkg
    rng = np.random.default_rng(91)
    n, ff, nexp, topk, T, layer = 512, 256, 6, 2, 5, 0
    nbk = lambda rows, cols, qt: rows * cols // qb.SHAPE[qt][0]
    gate, up = qb.random_blocks(rng, qb.Q4_K, nexp * nbk(ff, n, qb.Q4_K)), qb.random_blocks(rng, qb.Q4_K, nexp * nbk(ff, n, qb.Q4_K))
    down = qb.random_blocks(rng, qb.Q4_K, nexp * nbk(n, ff, qb.Q4_K))
    sgate, sup, sdown = (qb.random_blocks(rng, qb.Q8_0, nbk(r, c, qb.Q8_0)) for r, c in ((ff, n), (ff, n), (n, ff)))
    router = (rng.standard_normal((nexp, n)) * 0.05).astype(np.float32)
    srouter = (rng.standard_normal((1, n)) * 0.05).astype(np.float32)
    b = "blk.0."
    ts = [(b + "ffn_gate_inp.weight", gf.F32, [n, nexp], router.tobytes()), (b + "ffn_gate_inp_shexp.weight", gf.F32, [n, 1], srouter.tobytes()),
          (b + "ffn_gate_exps.weight", qb.Q4_K, [n, ff, nexp], gate), (b + "ffn_up_exps.weight", qb.Q4_K, [n, ff, nexp], up),
          (b + "ffn_down_exps.weight", qb.Q4_K, [ff, n, nexp], down), (b + "ffn_gate_shexp.weight", qb.Q8_0, [n, ff], sgate),
          (b + "ffn_up_shexp.weight", qb.Q8_0, [n, ff], sup), (b + "ffn_down_shexp.weight", qb.Q8_0, [ff, n], sdown)]
    path = gf.write(tmp_path / "mixed.gguf", ts)
    print("case gguf layer with Q4_K experts and a Q8_0 shared expert", flush=True)
    g = lib.fnx_gguf_open(path.encode())
    assert g, lib.fnx_last_error()
    z = pkg.MoeBufs()
    dev.ok(lib.fnx_gguf_moe_layer_bytes(g, layer, 0, ff, C.byref(z)))
    bufs = [dev.zeros(getattr(z, k + "_bytes"), t.uint8) for k in ("router", "gu", "down", "sh_gu", "sh_down")]
    for k, bf in zip(("router", "gu", "down", "sh_gu", "sh_down"), bufs):
        setattr(z, k, bf.data_ptr())
    L = pkg.MoeLayer()
    dev.ok(lib.fnx_gguf_load_moe_layer(g, layer, 0, ff, topk, C.byref(z), C.byref(L), dev.st()))
    dev.sync()
    lib.fnx_gguf_close(g)
    assert (L.gu.type, L.down.type, L.sh_gu.type, L.sh_down.type) == (qb.Q4_K, qb.Q4_K, qb.Q8_0, qb.Q8_0)
    gu_rb, dn_rb, sgu_rb, sdn_rb = n // 256 * 144, ff // 256 * 144, n // 32 * 34, ff // 32 * 34
    gu_w = np.concatenate([gate.reshape(nexp, ff * gu_rb), up.reshape(nexp, ff * gu_rb)], axis=1).reshape(-1)
    assert np.array_equal(bufs[1].cpu().numpy(), gu_w), "gate rows then up rows, expert by expert"
    # the window
    P = T * topk
    w = dict(xq=dev.zeros(T * (n // 32) * 36, t.uint8), logits=dev.zeros((T, nexp + 1), t.float32), topi=dev.zeros((T, topk), t.int32),
             topw=dev.zeros((T, topk), t.float32), jobs_gu=dev.zeros((P + 1) * 136, t.uint8), jobs_dn=dev.zeros((P + 1) * 136, t.uint8),
             njobs=dev.zeros(2, t.int32), gu=dev.zeros((P + T, 2 * ff), t.float32), part=dev.zeros((P + T, n), t.float32),
             sync=dev.zeros(pkg.MOE_SYNC_WORDS, t.int32))
    ws = pkg.MoeWs(*(w[k].data_ptr() for k in ("xq", "logits", "topi", "topw", "jobs_gu", "jobs_dn", "njobs", "gu", "part", "sync")))
    x = rng.standard_normal((T, n)).astype(np.float32)
    dx, out = dev.up(x), dev.zeros((T, n), t.float32)
    dev.ok(lib.fnx_moe_verify_layer(C.byref(L), dx.data_ptr(), T, out.data_ptr(), C.byref(ws), dev.st()))
    dev.sync()
    # the oracle's operators, in order
    W = np.concatenate([router, srouter])
    logits = oracle.gemv_f32(W, x)
    topi, topw = oracle.topk_logits(logits, nexp, topk)
    jg, jd = oracle.jobs(topi)
    xq = oracle.quantize_q8_1(x)
    gu = np.zeros((P + T, 2 * ff), np.float32)
    mm = oracle.lib.fnx_o_mmvq_type
    mm(qb.Q4_K, ol.ptr(gu_w), 2 * ff * gu_rb, 2 * ff, n, ol.ptr(np.ascontiguousarray(jg)), len(jg), ol.ptr(xq), ol.ptr(gu), 2 * ff, 8)
    sh = np.zeros(1, dtype=fnx_gpu.JOB_DTYPE)
    sh["n"][0] = T
    sh["y"][0, :T], sh["out"][0, :T] = np.arange(T), P + np.arange(T)
    sgu_w = np.concatenate([sgate, sup])
    mm(qb.Q8_0, ol.ptr(sgu_w), 0, 2 * ff, n, ol.ptr(sh), 1, ol.ptr(xq), ol.ptr(gu), 2 * ff, 8)
    hq = oracle.swiglu_stacked_q8_1(gu, ff)
    part = np.zeros((P + T, n), np.float32)
    mm(qb.Q4_K, ol.ptr(down), n * dn_rb, n, ff, ol.ptr(np.ascontiguousarray(jd)), len(jd), ol.ptr(hq), ol.ptr(part), n, 8)
    sh["y"][0, :T] = P + np.arange(T)
    mm(qb.Q8_0, ol.ptr(sdown), 0, n, ff, ol.ptr(sh), 1, ol.ptr(hq), ol.ptr(part), n, 8)
    want = oracle.moe_combine(part[:P], topw, part[P:], logits[:, nexp])
    assert np.array_equal(w["topi"].cpu().numpy(), topi)
    assert rel_l2(out.cpu().numpy(), want) <= 1e-3


def test_layer_with_a_q8_0_shared_expert_from_gguf(dev, oracle, tmp_path):
    """IQ3_S routed experts and a Q8_0 shared expert, the reference's own layer form (engine.cu:1600-1604): the loader
    re-lays the experts to unit64 and the shared expert's raw Q8_0 blocks to the split layout, and the window runs in
    its three launches plus the shared expert's dense ones."""
    import qtype_blocks as qb
    t, lib, pkg = dev.torch, dev.lib, dev.pkg
    rng = np.random.default_rng(93)
    n, ff, nexp, topk, T, layer = 2048, 512, 24, 10, 16, 3
    ts, a = gf.moe_layer_tensors(rng, layer, n, ff, nexp, fnx_gpu.random_iq3s)
    nbk = lambda rows, cols: rows * cols // 32
    sgate, sup, sdown = (qb.random_blocks(rng, qb.Q8_0, nbk(r, c)) for r, c in ((ff, n), (ff, n), (n, ff)))
    b = f"blk.{layer}."
    ts = ts[:5] + [(b + "ffn_gate_shexp.weight", qb.Q8_0, [n, ff], sgate), (b + "ffn_up_shexp.weight", qb.Q8_0, [n, ff], sup),
                   (b + "ffn_down_shexp.weight", qb.Q8_0, [ff, n], sdown)]
    path = gf.write(tmp_path / "q8shared.gguf", ts)
    print("case gguf layer with IQ3_S experts and a Q8_0 shared expert", flush=True)
    g = lib.fnx_gguf_open(path.encode())
    assert g, lib.fnx_last_error()
    z = pkg.MoeBufs()
    dev.ok(lib.fnx_gguf_moe_layer_bytes(g, layer, 0, ff, C.byref(z)))
    bufs = [dev.zeros(getattr(z, k + "_bytes"), t.uint8) for k in ("router", "gu", "down", "sh_gu", "sh_down")]
    for k, bf in zip(("router", "gu", "down", "sh_gu", "sh_down"), bufs):
        setattr(z, k, bf.data_ptr())
    L = pkg.MoeLayer()
    dev.ok(lib.fnx_gguf_load_moe_layer(g, layer, 0, ff, topk, C.byref(z), C.byref(L), dev.st()))
    dev.sync()
    lib.fnx_gguf_close(g)
    assert (L.gu.type, L.down.type) == (pkg.T_IQ3S_UNIT64, pkg.T_IQ3S_UNIT64)
    assert L.sh_gu_q8.q == bufs[3].data_ptr() and (L.sh_gu_q8.n_out, L.sh_gu_q8.n_in, L.sh_down_q8.n_out, L.sh_down_q8.n_in) == (2 * ff, n, n, ff)

    def split(raw, rows, cols):   # raw Q8_0 blocks (f16 d, 32 int8) -> the split arrays
        blk = raw.reshape(rows, cols // 32, 34)
        return np.ascontiguousarray(blk[:, :, 2:]).view(np.int8).reshape(rows, cols), np.ascontiguousarray(blk[:, :, :2]).view(np.uint16).reshape(rows, cols // 32)

    sh_q8 = (split(np.concatenate([sgate, sup]), 2 * ff, n), split(sdown, n, ff))
    got_q = bufs[3].cpu().numpy()
    assert np.array_equal(got_q[:2 * ff * n].view(np.int8).reshape(2 * ff, n), sh_q8[0][0]), "the split layout on the device: the values"
    assert np.array_equal(got_q[2 * ff * n:].view(np.uint16).reshape(2 * ff, n // 32), sh_q8[0][1]), "then the scales"
    gu = gf.slice_rows2(a["gate"], a["up"], n, ff, nexp, 0, ff)
    router = np.concatenate([a["router"], a["sh_router"]])
    x = rng.standard_normal((T, n)).astype(np.float32)
    want = oracle.moe_verify_layer(n, ff, nexp, topk, router, gu, a["down"], None, None, x, sh_q8=sh_q8)
    P = T * topk
    w = dict(xq=dev.zeros(T * (n // 32) * 36, t.uint8), logits=dev.zeros((T, nexp + 1), t.float32), topi=dev.zeros((T, topk), t.int32),
             topw=dev.zeros((T, topk), t.float32), jobs_gu=dev.zeros((P + 1) * 136, t.uint8), jobs_dn=dev.zeros((P + 1) * 136, t.uint8),
             njobs=dev.zeros(2, t.int32), gu=dev.zeros((P + T, 2 * ff), t.float32), part=dev.zeros((P + T, n), t.float32),
             sync=dev.zeros(pkg.MOE_SYNC_WORDS, t.int32))
    ws = pkg.MoeWs(*(w[k].data_ptr() for k in ("xq", "logits", "topi", "topw", "jobs_gu", "jobs_dn", "njobs", "gu", "part", "sync")))
    dx, out = dev.up(x), dev.zeros((T, n), t.float32)
    dev.ok(lib.fnx_moe_verify_layer(C.byref(L), dx.data_ptr(), T, out.data_ptr(), C.byref(ws), dev.st()))
    dev.sync()
    assert np.array_equal(w["topi"].cpu().numpy(), want["topi"]) and int(w["njobs"][0].item()) == want["njobs"]
    assert rel_l2(out.cpu().numpy(), want["out"]) <= 1e-3

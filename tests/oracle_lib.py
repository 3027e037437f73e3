"""ctypes binding of the CPU oracle (oracle/liboracle.so) for the tests, the smoke check and the benchmark's CPU leg.

The oracle is the checker, never the product: nothing in the device library or its host mirror imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
MAXT = 16
IQ3S_BLOCK = 110
Q8_1_BLOCK = 36


class Job(C.Structure):
    _fields_ = [("w", C.c_int), ("n", C.c_int), ("y", C.c_int * MAXT), ("out", C.c_int * MAXT)]


class MoeLayer(C.Structure):
    _fields_ = [("n", C.c_int), ("ff", C.c_int), ("nexp", C.c_int), ("topk", C.c_int), ("router", C.c_void_p),
                ("gu", C.c_void_p), ("down", C.c_void_p), ("sh_gu", C.c_void_p), ("sh_down", C.c_void_p),
                ("sh_gu_q", C.c_void_p), ("sh_gu_d", C.c_void_p), ("sh_down_q", C.c_void_p), ("sh_down_d", C.c_void_p)]


JOB_DTYPE = np.dtype([("w", "<i4"), ("n", "<i4"), ("y", "<i4", (MAXT,)), ("out", "<i4", (MAXT,))])


def _build():
    subprocess.run(["make", "-C", ORACLE_DIR, "all"], check=True, capture_output=True)


def load():
    path = os.path.join(ORACLE_DIR, "liboracle.so")
    if not os.path.exists(path):
        _build()
    lib = C.CDLL(path)
    vp, i, f, sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t
    sig = {
        "fnx_o_h2f": (f, [C.c_uint16]),
        "fnx_o_f2h": (C.c_uint16, [f]),
        "fnx_o_f2h_rn": (C.c_uint16, [f]),
        "fnx_o_dp4a": (i, [i, i, i]),
        "fnx_o_expf": (None, [vp, C.c_size_t, vp]),
        "fnx_o_iq3s_dequant": (None, [vp, sz, vp]),
        "fnx_o_iq3s_quantize": (None, [vp, sz, vp]),
        "fnx_o_quantize_q8_1": (None, [vp, vp, i, i]),
        "fnx_o_vec_dot_iq3s_q8_1": (f, [vp, vp, i]),
        "fnx_o_mmvq_iq3s": (None, [vp, sz, vp, i, i, vp, i, vp, vp, i, i]),
        "fnx_o_gemv_exact": (None, [vp, i, i, vp, i, vp]),
        "fnx_o_gemv_f32": (None, [vp, vp, vp, i, i, i]),
        "fnx_o_gemv_bf16": (None, [vp, vp, vp, i, i, i]),
        "fnx_o_topk_logits": (None, [vp, i, i, i, i, vp, vp]),
        "fnx_o_topk_softmax": (None, [vp, i, i, i, i, vp, vp]),
        "fnx_o_jobs": (i, [vp, i, i, vp, vp]),
        "fnx_o_swiglu_q8_1": (None, [vp, vp, vp, i, i]),
        "fnx_o_swiglu_stacked_q8_1": (None, [vp, vp, i, i]),
        "fnx_o_moe_combine": (None, [vp, vp, vp, vp, i, vp, i, i, i]),
        "fnx_o_argmax": (C.c_uint, [vp, i, i, i, vp, vp]),
        "fnx_o_lookup_drafts": (i, [vp, i, i, i, i, vp, vp]),
        "fnx_o_lookup_fixed": (i, [vp, i, i, i, i, vp]),
        "fnx_o_accept_greedy": (i, [vp, vp, i]),
        "fnx_o_type_block": (i, [C.c_uint32, vp, vp]),
        "fnx_o_dequant": (None, [C.c_uint32, vp, sz, vp]),
        "fnx_o_vec_dot_type": (f, [C.c_uint32, vp, i, vp]),
        "fnx_o_mmvq_type": (None, [C.c_uint32, vp, sz, i, i, vp, i, vp, vp, i, i]),
        "fnx_o_top_tokens": (C.c_uint, [vp, i, i, i, vp, vp, vp, i, vp, vp, vp, vp, vp, vp, vp]),
        "fnx_o_penalize_row": (None, [vp, i, vp, vp]),
        "fnx_o_make_dist": (i, [vp, vp, i, f, f, f, i, vp, vp]),
        "fnx_o_draw": (i, [vp, vp, i, C.c_double]),
        "fnx_o_accept_sampled": (i, [vp, vp, i, i, vp, f, f, f, i, vp, vp, vp, i, vp, vp, vp]),
        "fnx_o_pf_jobs": (i, [vp, i, i, i, i, vp, vp, vp]),
        "fnx_o_moe_verify_layer": (None, [vp, vp, i, vp, vp, vp, vp, vp, i]),
        "fnx_o_iq3s_dequant_f16": (None, [vp, sz, vp]),
        "fnx_o_f32_f16": (None, [vp, sz, vp]),
        "fnx_o_moe_mma": (None, [vp, sz, i, i, vp, i, i, vp, i, vp, i]),
        "fnx_o_swiglu_h16": (None, [vp, i, i, vp]),
        "fnx_o_moe_prefill_layer": (None, [vp, vp, i, i, vp, vp, vp, vp, vp, i]),
        "fnx_o_rms_norm_rows": (None, [vp, vp, vp, i, i, f]),
        "fnx_o_quantize_q8_0_split": (None, [vp, i, i, vp, vp]),
        "fnx_o_q8s_gemv": (None, [vp, vp, i, i, vp, vp, i, i]),
        "fnx_o_attn_prep_append": (None, [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, f, vp]),
        "fnx_o_attn": (None, [vp, vp, vp, vp, i, i, i, i, i]),
        "fnx_o_rng_init": (None, [vp, C.c_ulonglong]),
        "fnx_o_rng_next": (C.c_uint, [vp]),
        "fnx_o_threads": (i, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def load_ref():
    """The reference's own tensor_convert.hpp and GGUF reader compiled as a shared library, or None when it was not built."""
    path = os.path.join(ORACLE_DIR, "_ref", "libfnx_ref.so")
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path)
    lib.fnx_ref_h2f.restype = C.c_float
    lib.fnx_ref_h2f.argtypes = [C.c_uint16]
    lib.fnx_ref_f2h.restype = C.c_uint16
    lib.fnx_ref_f2h.argtypes = [C.c_float]
    lib.fnx_ref_iq3s_grid.restype = C.POINTER(C.c_uint32)
    lib.fnx_ref_dequantize.restype = C.c_int
    lib.fnx_ref_dequantize.argtypes = [C.c_uint32, C.c_void_p, C.c_size_t, C.c_void_p]
    if hasattr(lib, "fnx_ref_gguf_open"):   # the reference's GGUF reader (a library built before it was added lacks it)
        lib.fnx_ref_gguf_open.restype = C.c_void_p
        lib.fnx_ref_gguf_open.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t]
        lib.fnx_ref_gguf_close.restype = None
        lib.fnx_ref_gguf_close.argtypes = [C.c_void_p]
        for name in ("fnx_ref_gguf_count", "fnx_ref_gguf_shards"):
            getattr(lib, name).restype = C.c_int
            getattr(lib, name).argtypes = [C.c_void_p]
        lib.fnx_ref_gguf_tensor.restype = C.c_int
        lib.fnx_ref_gguf_tensor.argtypes = [C.c_void_p, C.c_int, C.c_char_p, C.c_size_t, C.POINTER(C.c_int64)]
        lib.fnx_ref_gguf_data.restype = C.c_void_p
        lib.fnx_ref_gguf_data.argtypes = [C.c_void_p, C.c_char_p]
        lib.fnx_ref_gguf_has_key.restype = C.c_int
        lib.fnx_ref_gguf_has_key.argtypes = [C.c_void_p, C.c_char_p]
        lib.fnx_ref_gguf_num.restype = C.c_int
        lib.fnx_ref_gguf_num.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_double)]
        lib.fnx_ref_gguf_str.restype = C.c_int
        lib.fnx_ref_gguf_str.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_size_t]
    return lib


def ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


class Oracle:
    """numpy-level helpers over the C oracle."""

    def __init__(self):
        self.lib = load()

    # ---- formats
    def iq3s_quantize(self, w):
        w = np.ascontiguousarray(w, dtype=np.float32)
        assert w.size % 256 == 0
        out = np.zeros(w.size // 256 * IQ3S_BLOCK, dtype=np.uint8)
        self.lib.fnx_o_iq3s_quantize(ptr(w), w.size, ptr(out))
        return out

    def expf(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty_like(x)
        self.lib.fnx_o_expf(ptr(x), x.size, ptr(out))
        return out

    def iq3s_dequant(self, blocks):
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        n = blocks.size // IQ3S_BLOCK * 256
        out = np.empty(n, dtype=np.float32)
        self.lib.fnx_o_iq3s_dequant(ptr(blocks), n, ptr(out))
        return out

    def quantize_q8_1(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, n = x.shape
        q = np.zeros(rows * (n // 32) * Q8_1_BLOCK, dtype=np.uint8)
        self.lib.fnx_o_quantize_q8_1(ptr(x), ptr(q), n, rows)
        return q

    # ---- mat-vec
    def mmvq(self, w, w_stride, nrows, ncols, jobs, yq, out_rows, threads=8):
        out = np.zeros((out_rows, nrows), dtype=np.float32)
        jobs = np.ascontiguousarray(jobs)
        self.lib.fnx_o_mmvq_iq3s(ptr(w), w_stride, None, nrows, ncols, ptr(jobs), len(jobs), ptr(yq), ptr(out), nrows, threads)
        return out

    def gemv_iq3s(self, w, nrows, ncols, x, threads=8):
        """x f32 [T][ncols] -> [T][nrows] through q8_1, T <= 16 per job"""
        T = x.shape[0]
        yq = self.quantize_q8_1(x)
        out = np.zeros((T, nrows), dtype=np.float32)
        for t0 in range(0, T, MAXT):
            nt = min(MAXT, T - t0)
            job = np.zeros(1, dtype=JOB_DTYPE)
            job["n"] = nt
            job["y"][0, :nt] = np.arange(t0, t0 + nt)
            job["out"][0, :nt] = np.arange(t0, t0 + nt)
            self.lib.fnx_o_mmvq_iq3s(ptr(w), 0, None, nrows, ncols, ptr(job), 1, ptr(yq), ptr(out), nrows, threads)
        return out

    def gemv_exact(self, w, nrows, ncols, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        T = x.shape[0]
        out = np.zeros((T, nrows), dtype=np.float64)
        self.lib.fnx_o_gemv_exact(ptr(w), nrows, ncols, ptr(x), T, ptr(out))
        return out

    def gemv_f32(self, W, x):
        W = np.ascontiguousarray(W, dtype=np.float32)
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, n = W.shape
        T = x.shape[0]
        y = np.zeros((T, rows), dtype=np.float32)
        self.lib.fnx_o_gemv_f32(ptr(W), ptr(x), ptr(y), rows, n, T)
        return y

    def gemv_bf16(self, W, x):
        W = np.ascontiguousarray(W, dtype=np.uint16)
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, n = W.shape
        T = x.shape[0]
        y = np.zeros((T, rows), dtype=np.float32)
        self.lib.fnx_o_gemv_bf16(ptr(W), ptr(x), ptr(y), rows, n, T)
        return y

    # ---- routing
    def topk_logits(self, logits, nexp, topk):
        logits = np.ascontiguousarray(logits, dtype=np.float32)
        T, stride = logits.shape
        topi = np.zeros((T, topk), dtype=np.int32)
        topw = np.zeros((T, topk), dtype=np.float32)
        self.lib.fnx_o_topk_logits(ptr(logits), stride, T, nexp, topk, ptr(topi), ptr(topw))
        return topi, topw

    def topk_softmax(self, logits, nexp, topk):
        logits = np.ascontiguousarray(logits, dtype=np.float32)
        T, stride = logits.shape
        topi = np.zeros((T, topk), dtype=np.int32)
        topw = np.zeros((T, topk), dtype=np.float32)
        self.lib.fnx_o_topk_softmax(ptr(logits), stride, T, nexp, topk, ptr(topi), ptr(topw))
        return topi, topw

    def jobs(self, topi):
        topi = np.ascontiguousarray(topi, dtype=np.int32)
        T, topk = topi.shape
        gu = np.zeros(T * topk, dtype=JOB_DTYPE)
        dn = np.zeros(T * topk, dtype=JOB_DTYPE)
        nj = self.lib.fnx_o_jobs(ptr(topi), T, topk, ptr(gu), ptr(dn))
        return gu[:nj], dn[:nj]

    def swiglu_stacked_q8_1(self, gu, ffs):
        gu = np.ascontiguousarray(gu, dtype=np.float32)
        rows = gu.shape[0]
        hq = np.zeros(rows * (ffs // 32) * Q8_1_BLOCK, dtype=np.uint8)
        self.lib.fnx_o_swiglu_stacked_q8_1(ptr(gu), ptr(hq), ffs, rows)
        return hq

    def swiglu_q8_1(self, g, u):
        g = np.ascontiguousarray(g, dtype=np.float32)
        u = np.ascontiguousarray(u, dtype=np.float32)
        rows, n = g.shape
        q = np.zeros(rows * (n // 32) * Q8_1_BLOCK, dtype=np.uint8)
        self.lib.fnx_o_swiglu_q8_1(ptr(g), ptr(u), ptr(q), n, rows)
        return q

    def moe_combine(self, part, topw, sh, sh_logit):
        part = np.ascontiguousarray(part, dtype=np.float32)
        topw = np.ascontiguousarray(topw, dtype=np.float32)
        sh = np.ascontiguousarray(sh, dtype=np.float32)
        sh_logit = np.ascontiguousarray(sh_logit, dtype=np.float32)
        T, topk = topw.shape
        n = part.shape[1]
        out = np.zeros((T, n), dtype=np.float32)
        self.lib.fnx_o_moe_combine(ptr(part), ptr(topw), ptr(sh), ptr(sh_logit), 1, ptr(out), T, n, topk)
        return out

    # ---- head / drafting
    def argmax(self, logits, v0=0):
        logits = np.ascontiguousarray(logits, dtype=np.float32)
        T, rows = logits.shape
        bv = np.zeros(T, dtype=np.float32)
        bi = np.zeros(T, dtype=np.int32)
        err = self.lib.fnx_o_argmax(ptr(logits), rows, T, v0, ptr(bv), ptr(bi))
        return bv, bi, err

    def lookup_drafts(self, ctx, lk, d1, key_n=3):
        ctx = np.ascontiguousarray(ctx, dtype=np.int32)
        out = np.zeros(max(lk, 1) + 8, dtype=np.int32)
        match = C.c_int(-1)
        n = self.lib.fnx_o_lookup_drafts(ptr(ctx), len(ctx), key_n, lk, d1, ptr(out), C.byref(match))
        return out[:n].copy(), match.value

    def lookup_fixed(self, ctx, lk, d1, key_n=3):
        ctx = np.ascontiguousarray(ctx, dtype=np.int32)
        out = np.zeros(max(lk, 1) + 8, dtype=np.int32)
        n = self.lib.fnx_o_lookup_fixed(ptr(ctx), len(ctx), key_n, lk, d1, ptr(out))
        return out[:n].copy()

    def accept_greedy(self, rows, o):
        rows = np.ascontiguousarray(rows, dtype=np.int32)
        o = np.ascontiguousarray(o, dtype=np.int32)
        return self.lib.fnx_o_accept_greedy(ptr(rows), ptr(o), len(rows))

    def pf_jobs(self, topi, nexp, pf_job):
        topi = np.ascontiguousarray(topi, dtype=np.int32)
        Cn, topk = topi.shape
        js = 2 + 2 * pf_job
        cap = Cn * topk // pf_job + nexp + 1
        gu = np.zeros((cap, js), dtype=np.int32)
        dn = np.zeros((cap, js), dtype=np.int32)
        cnt = np.zeros(nexp, dtype=np.int32)
        nj = self.lib.fnx_o_pf_jobs(ptr(topi), Cn, topk, nexp, pf_job, ptr(gu), ptr(dn), ptr(cnt))
        return gu[:nj], dn[:nj], cnt

    # ---- the prompt path
    def iq3s_dequant_f16(self, blocks):
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        n = blocks.size // IQ3S_BLOCK * 256
        out = np.empty(n, dtype=np.float16)
        self.lib.fnx_o_iq3s_dequant_f16(ptr(blocks), n, ptr(out))
        return out

    def f32_f16(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape, dtype=np.float16)
        self.lib.fnx_o_f32_f16(ptr(x), x.size, ptr(out))
        return out

    def moe_mma(self, w, w_stride, nrows, ncols, jobs, pf_job, x16, out_rows, out=None, threads=8):
        """jobs: int32 [njobs][2 + 2 pf_job]; x16: float16 [rows][ldx]"""
        jobs = np.ascontiguousarray(jobs, dtype=np.int32)
        x16 = np.ascontiguousarray(x16, dtype=np.float16)
        if out is None:
            out = np.zeros((out_rows, nrows), dtype=np.float32)
        self.lib.fnx_o_moe_mma(ptr(w), w_stride, nrows, ncols, ptr(jobs), len(jobs), pf_job, ptr(x16), x16.shape[1], ptr(out), threads)
        return out

    def swiglu_h16(self, gu, ffs):
        gu = np.ascontiguousarray(gu, dtype=np.float32)
        out = np.empty((gu.shape[0], ffs), dtype=np.float16)
        self.lib.fnx_o_swiglu_h16(ptr(gu), ffs, gu.shape[0], ptr(out))
        return out

    def moe_prefill_layer(self, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x, pf_job=64, threads=8):
        router = np.ascontiguousarray(router, dtype=np.float32)
        x = np.ascontiguousarray(x, dtype=np.float32)
        Cn = x.shape[0]
        L = MoeLayer(n, ff, nexp, topk, ptr(router), ptr(gu), ptr(down), ptr(sh_gu), ptr(sh_down))
        out = np.zeros((Cn, n), dtype=np.float32)
        logits = np.zeros((Cn, nexp + 1), dtype=np.float32)
        topi = np.zeros((Cn, topk), dtype=np.int32)
        topw = np.zeros((Cn, topk), dtype=np.float32)
        nj = C.c_int(0)
        self.lib.fnx_o_moe_prefill_layer(C.byref(L), ptr(x), Cn, pf_job, ptr(out), ptr(logits), ptr(topi), ptr(topw), C.byref(nj), threads)
        return dict(out=out, logits=logits, topi=topi, topw=topw, njobs=nj.value)

    # ---- the layer
    def moe_verify_layer(self, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, x, threads=8, sh_q8=None):
        """sh_q8: the shared expert as split Q8_0 instead: ((q, d) of gate|up, (q, d) of down); sh_gu / sh_down may then be None"""
        router = np.ascontiguousarray(router, dtype=np.float32)
        x = np.ascontiguousarray(x, dtype=np.float32)
        T = x.shape[0]
        L = MoeLayer(n, ff, nexp, topk, ptr(router), ptr(gu), ptr(down), ptr(sh_gu), ptr(sh_down))
        if sh_q8 is not None:
            L.sh_gu_q, L.sh_gu_d, L.sh_down_q, L.sh_down_d = ptr(sh_q8[0][0]), ptr(sh_q8[0][1]), ptr(sh_q8[1][0]), ptr(sh_q8[1][1])
        out = np.zeros((T, n), dtype=np.float32)
        logits = np.zeros((T, nexp + 1), dtype=np.float32)
        topi = np.zeros((T, topk), dtype=np.int32)
        topw = np.zeros((T, topk), dtype=np.float32)
        nj = C.c_int(0)
        self.lib.fnx_o_moe_verify_layer(C.byref(L), ptr(x), T, ptr(out), ptr(logits), ptr(topi), ptr(topw), C.byref(nj), threads)
        return dict(out=out, logits=logits, topi=topi, topw=topw, njobs=nj.value)

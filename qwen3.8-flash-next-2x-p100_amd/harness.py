"""Host-side harness over the C ABI: numpy arrays in and out through torch device buffers on the current stream, the
operators one by one, whole layers (verify window, prompt chunk) and a whole decoder with its caches and workspace, and a
synthetic model of a given shape with random weights in the library's formats. The benchmark and the tests drive the
library through these classes; nothing here computes a result of its own."""
import ctypes as C
import sys

import numpy as np

HD = 256   # head width (model.hpp:41 of the reference)


def random_iq3s(rng, nblocks, dmax=3e-4, raw_bytes=False):
    """valid IQ3_S blocks with uniformly random codes, signs and scales (any byte pattern is a valid block).
    raw_bytes: the generator's byte stream as it comes (other values than the default draws; much faster for gigabytes)"""
    if raw_bytes:
        b = rng.integers(0, 1 << 64, size=(nblocks * 110 + 7) // 8, dtype=np.uint64).view(np.uint8)[:nblocks * 110].reshape(nblocks, 110)
    else:
        b = rng.integers(0, 256, size=(nblocks, 110), dtype=np.uint8)
    d = (rng.random(nblocks) * dmax + 1e-5).astype(np.float16)
    b[:, 0:2] = d.view(np.uint8).reshape(nblocks, 2)
    return b.reshape(-1)


def q8s_draw(rng, quantize, rows, cols, scale, cheap=False):
    """a split-Q8_0 matrix (int8 values, f16 block scales) with entries of standard deviation `scale`: Gaussian weights
    through quantize(w) -> (q, d), or (cheap) uniformly random int8 values under block scales of scale / 74 with a random
    last mantissa nibble (every (q, d) pair is a valid matrix; no float matrix is drawn)"""
    if cheap:
        q = rng.integers(0, 1 << 64, size=rows * cols // 8, dtype=np.uint64).view(np.int8).reshape(rows, cols)
        d0 = np.array([scale / 74.0], dtype=np.float16).view(np.uint16)[0] & np.uint16(0xFFF0)
        d = d0 | rng.integers(0, 16, (rows, cols // 32), dtype=np.uint16)
        return q, d
    if quantize is None:
        raise ValueError("Gaussian draws need a Q8_0 quantiser; pass quantize or cheap_draws=True")
    return quantize((rng.standard_normal((rows, cols)) * scale).astype(np.float32))


class SyntheticDecoder:
    def __init__(self, quantize=None, seed=1, n=256, nq=4, nkv=2, nlayers=2, vocab=1000, max_ctx=128, nexp=8, topk=2, ff=256, rope_scaled=False,
                 cyclic=False, cheap_draws=False):
        """quantize: w (rows x cols float32) -> (int8 values, f16 block scales as uint16), the split-Q8_0 quantiser for
        Gaussian draws (none is needed with cheap_draws).
        cheap_draws: cheaper draws for full-size models (other values than the default draws): the dense matrices as random
        int8 values, the embedding as f16 bit patterns, the IQ3_S blocks from the generator's 64-bit stream.
        cyclic: a model whose pick depends on the row's token alone (the attention's output projections are zero) and
        whose draft layer is the model's single layer behind an identity projection of the embedding, so greedy decoding
        runs into a cycle, the draft layer mostly predicts the next token, prompt lookup fires and drafts are kept."""
        rng = np.random.default_rng(seed)
        _q8s = lambda rng, _, rows, cols, scale: q8s_draw(rng, quantize, rows, cols, scale, cheap_draws)
        self.cfg = dict(n=n, nq=nq, nkv=nkv, nlayers=nlayers, vocab=vocab, max_ctx=max_ctx, nexp=nexp, topk=topk, ff=ff, eps=1e-6)
        self.rope = (1e7, 0, 0.0, 0.0, 1.0, 1.0) if not rope_scaled else (1e4, 1, 4.0, 20.0, 0.25, 1.0 + 0.1 * np.log(4.0))
        nb = lambda rows, cols: rows * cols // 256
        sw = 1.0 / np.sqrt(n)
        iq3s = lambda nblocks: random_iq3s(rng, nblocks, dmax=4e-4, raw_bytes=cheap_draws)

        def layer():
            L = dict(attn_norm=(1 + 0.1 * rng.standard_normal(n)).astype(np.float32), q_norm=(1 + 0.1 * rng.standard_normal(HD)).astype(np.float32),
                     k_norm=(1 + 0.1 * rng.standard_normal(HD)).astype(np.float32), ffn_norm=(1 + 0.1 * rng.standard_normal(n)).astype(np.float32),
                     wq=_q8s(rng, None, nq * 2 * HD, n, sw), wk=_q8s(rng, None, nkv * HD, n, sw), wv=_q8s(rng, None, nkv * HD, n, sw),
                     wo=_q8s(rng, None, n, nq * HD, 1.0 / np.sqrt(nq * HD)),
                     router=(rng.standard_normal((nexp + 1, n)) * 0.05).astype(np.float32),
                     gu=iq3s(nexp * nb(2 * ff, n)), down=iq3s(nexp * nb(n, ff)),
                     sh_gu=iq3s(nb(2 * ff, n)), sh_down=iq3s(nb(n, ff)))
            return L

        self.layers = [layer() for _ in range(nlayers)]
        self.out_norm = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
        self.head = _q8s(rng, None, vocab, n, sw)
        if cheap_draws:   # f16 bit patterns drawn directly: a random sign, exponent field 12..15 (magnitudes 1/8 .. 2), random mantissa
            self.emb = ((rng.integers(0, 1 << 16, (vocab, n), dtype=np.uint16) & np.uint16(0x8FFF)) | np.uint16(0x3000)).view(np.float16)
        else:
            self.emb = rng.standard_normal((vocab, n)).astype(np.float16)
        self.mtp = dict(norm_emb=(1 + 0.1 * rng.standard_normal(n)).astype(np.float32), norm_hid=(1 + 0.1 * rng.standard_normal(n)).astype(np.float32),
                        out_norm=(1 + 0.1 * rng.standard_normal(n)).astype(np.float32), fc_emb=_q8s(rng, None, n, n, sw),
                        fc_hid=_q8s(rng, None, n, n, sw), head=_q8s(rng, None, vocab, n, sw), layer=layer())
        if cyclic:
            assert nlayers == 1
            zero = lambda t: (np.zeros_like(t[0]), np.zeros_like(t[1]))
            self.layers[0]["wo"] = zero(self.layers[0]["wo"])
            e = self.emb.astype(np.float32)
            self.emb = (e / np.sqrt((e * e).mean(axis=1, keepdims=True))).astype(np.float16)
            eye_q, eye_d = quantize(np.eye(n, dtype=np.float32))
            self.mtp = dict(norm_emb=np.ones(n, dtype=np.float32), norm_hid=self.mtp["norm_hid"], out_norm=self.out_norm, fc_emb=(eye_q, eye_d),
                            fc_hid=zero(self.mtp["fc_hid"]), head=self.head, layer=self.layers[0])


JOB_DTYPE = np.dtype([("w", "<i4"), ("n", "<i4"), ("y", "<i4", (16,)), ("out", "<i4", (16,))])


V_BLOCK = 8   # positions of a dimension that lie together in the library's V cache


def v_blocked(vc):
    """[pos][nkv][256] -> the library's V cache layout [pos / 8][nkv][256][pos % 8] (pos a multiple of 8)"""
    p, nkv, hd = vc.shape
    return np.ascontiguousarray(vc.reshape(p // V_BLOCK, V_BLOCK, nkv, hd).transpose(0, 2, 3, 1))


def v_rows(vb):
    """the inverse of v_blocked"""
    b, nkv, hd, _ = vb.shape
    return np.ascontiguousarray(vb.transpose(0, 3, 1, 2)).reshape(b * V_BLOCK, nkv, hd)


def pad4(a):
    """rows up to a whole block of the V cache"""
    extra = (-a.shape[0]) % V_BLOCK
    return a if not extra else np.concatenate([a, np.zeros((extra,) + a.shape[1:], dtype=a.dtype)])


class Dev:
    """numpy in, numpy out, through device memory and the C ABI on the current torch stream"""

    def __init__(self):
        import torch
        self.torch = torch
        self.pkg = sys.modules[__package__]
        self.lib = self.pkg.lib()
        self.dev = torch.device("cuda:0")

    def up(self, a):
        t = self.torch.from_numpy(np.ascontiguousarray(a))
        return t.to(self.dev)

    def zeros(self, shape, dtype):
        return self.torch.zeros(shape, dtype=dtype, device=self.dev)

    def st(self):
        return self.pkg.stream_ptr()

    def ok(self, status):
        self.pkg.check(status)

    def sync(self):
        self.torch.cuda.synchronize()

    # ---- operators
    def quantize_q8_1(self, x):
        t = self.torch
        rows, n = x.shape
        dx = self.up(x.astype(np.float32))
        q = self.zeros(rows * (n // 32) * 36, t.uint8)
        self.ok(self.lib.fnx_quantize_q8_1(dx.data_ptr(), q.data_ptr(), n, rows, self.st()))
        self.sync()
        return q.cpu().numpy()

    def gemv(self, W, x, bf16=False):
        t = self.torch
        rows, n = W.shape
        T = x.shape[0]
        dW, dx = self.up(W), self.up(x.astype(np.float32))
        y = self.zeros((T, rows), t.float32)
        fn = self.lib.fnx_gemv_bf16 if bf16 else self.lib.fnx_gemv_f32
        self.ok(fn(dW.data_ptr(), dx.data_ptr(), y.data_ptr(), rows, n, T, self.st()))
        self.sync()
        return y.cpu().numpy()

    def repack(self, w, in_place=True):
        """raw IQ3_S blocks (numpy) -> unit64 bytes (numpy), through the device"""
        t = self.torch
        src = self.up(w)
        dst = src if in_place else self.zeros(src.numel(), t.uint8)
        self.ok(self.lib.fnx_iq3s_repack(src.data_ptr(), dst.data_ptr(), w.size // 110 * 256, self.st()))
        self.sync()
        return dst.cpu().numpy()

    def mmvq(self, w, w_stride, nrows, ncols, jobs, yq, out_rows, njobs_dev=True, packed=False, tile16=False):
        """tile16: the matrices re-laid a second time into the prompt path's layout (w_stride then counts that layout's bytes)"""
        t = self.torch
        dw_, dj, dy = self.up(w), self.up(jobs.view(np.uint8).reshape(-1)), self.up(yq)
        if packed or tile16:
            self.ok(self.lib.fnx_iq3s_repack(dw_.data_ptr(), dw_.data_ptr(), w.size // 110 * 256, self.st()))
        out = self.zeros((out_rows, nrows), t.float32)
        W = W0 = self.pkg.dw(dw_, ncols, nrows, packed=packed)
        w_stride0 = w_stride
        if tile16:
            nmat = w.size // (nrows * (ncols // 256) * 110)
            one = self.lib.fnx_iq3s_tile16_bytes(nrows, ncols, 1)
            assert one > 0
            d16 = self.zeros(one * nmat, t.uint8)
            self.ok(self.lib.fnx_iq3s_tile16(dw_.data_ptr(), d16.data_ptr(), nrows, ncols, nmat, self.st()))
            W = self.pkg.dw(d16, ncols, nrows, tile16=True)
            w_stride = one if w_stride else 0
            self._keep = d16
        nj = self.up(np.array([len(jobs)], dtype=np.int32))
        self.ok(self.lib.fnx_mmvq(C.byref(W), w_stride, dj.data_ptr(), nj.data_ptr() if njobs_dev else None, len(jobs), dy.data_ptr(),
                                  out.data_ptr(), nrows, self.st()))
        self.sync()
        return out.cpu().numpy()

    def gemv_iq3s(self, w, nrows, ncols, x, packed=False, tile16=False):
        T = x.shape[0]
        yq = self.quantize_q8_1(x)
        jobs = np.zeros((T + 15) // 16, dtype=JOB_DTYPE)
        for j in range(len(jobs)):
            nt = min(16, T - 16 * j)
            jobs["n"][j] = nt
            jobs["y"][j, :nt] = np.arange(16 * j, 16 * j + nt)
            jobs["out"][j, :nt] = np.arange(16 * j, 16 * j + nt)
        return self.mmvq(w, 0, nrows, ncols, jobs, yq, T, packed=packed, tile16=tile16)

    def route(self, logits, nexp, topk, fused_W=None, x=None, bf16=False):
        t = self.torch
        T = logits.shape[0] if logits is not None else x.shape[0]
        P = T * topk
        topi = self.zeros((T, topk), t.int32)
        topw = self.zeros((T, topk), t.float32)
        gu = self.zeros((P + 1) * 136, t.uint8)
        dn = self.zeros((P + 1) * 136, t.uint8)
        nj = self.zeros(2, t.int32)
        if fused_W is None:
            dl = self.up(logits.astype(np.float32))
            self.ok(self.lib.fnx_route(dl.data_ptr(), logits.shape[1], T, nexp, topk, topi.data_ptr(), topw.data_ptr(), gu.data_ptr(),
                                       dn.data_ptr(), nj.data_ptr(), self.st()))
            lg = None
        else:
            dW, dx = self.up(fused_W), self.up(x.astype(np.float32))
            dl = self.zeros((T, nexp + 1), t.float32)
            self.ok(self.lib.fnx_router_route(dW.data_ptr(), int(bf16), dx.data_ptr(), dl.data_ptr(), T, x.shape[1], nexp, topk,
                                              topi.data_ptr(), topw.data_ptr(), gu.data_ptr(), dn.data_ptr(), nj.data_ptr(), self.st()))
            lg = dl
        self.sync()
        njh = nj.cpu().numpy()
        n = int(njh[0])
        return dict(topi=topi.cpu().numpy(), topw=topw.cpu().numpy(), njobs=njh,
                    gu=gu.cpu().numpy()[:n * 136].view(JOB_DTYPE), dn=dn.cpu().numpy()[:n * 136].view(JOB_DTYPE),
                    logits=None if lg is None else lg.cpu().numpy())

    def argmax(self, logits, v0=0):
        t = self.torch
        T, rows = logits.shape
        dl = self.up(logits.astype(np.float32))
        bv, bi = self.zeros(T, t.float32), self.zeros(T, t.int32)
        keys, err = self.zeros(self.pkg.ARGMAX_WORDS, t.int64), self.zeros(1, t.int32)
        self.ok(self.lib.fnx_argmax(dl.data_ptr(), rows, T, v0, bv.data_ptr(), bi.data_ptr(), keys.data_ptr(), err.data_ptr(), self.st()))
        self.sync()
        assert int(keys.abs().sum().item()) == 0, "argmax leaves its keys at zero"
        return bv.cpu().numpy(), bi.cpu().numpy(), int(err.item())

    def lookup(self, ctx, lk, d1, key_n=3):
        t = self.torch
        dc = self.up(np.asarray(ctx, dtype=np.int32)) if len(ctx) else self.zeros(1, t.int32)
        dd = self.up(np.array([d1], dtype=np.int32))
        out, n_out, match = self.zeros(max(lk, 1), t.int32), self.zeros(1, t.int32), self.zeros(1, t.int32)
        self.ok(self.lib.fnx_lookup_drafts_dev(dc.data_ptr(), len(ctx), key_n, lk, dd.data_ptr(), out.data_ptr(), n_out.data_ptr(),
                                               match.data_ptr(), self.st()))
        self.sync()
        n = int(n_out.item())
        return out.cpu().numpy()[:n], int(match.item())

    def accept(self, rows, o):
        t = self.torch
        dr, do = self.up(np.asarray(rows, dtype=np.int32)), self.up(np.asarray(o, dtype=np.int32))
        n = self.zeros(1, t.int32)
        self.ok(self.lib.fnx_accept_greedy_dev(dr.data_ptr(), do.data_ptr(), len(rows), n.data_ptr(), self.st()))
        self.sync()
        return int(n.item())


    # ---- the prompt path
    def pf_route(self, logits, nexp, topk):
        t = self.torch
        Cn = logits.shape[0]
        P, cap = Cn * topk, Cn * topk // 64 + nexp
        dl = self.up(logits.astype(np.float32))
        topi, topw = self.zeros((Cn, topk), t.int32), self.zeros((Cn, topk), t.float32)
        cnt, jbase, nj = self.zeros(nexp, t.int32), self.zeros(nexp, t.int32), self.zeros(2, t.int32)
        gu, dn = self.zeros((cap, 130), t.int32), self.zeros((cap, 130), t.int32)
        self.ok(self.lib.fnx_pf_route(dl.data_ptr(), logits.shape[1], Cn, nexp, topk, topi.data_ptr(), topw.data_ptr(), cnt.data_ptr(),
                                      jbase.data_ptr(), gu.data_ptr(), dn.data_ptr(), cap, nj.data_ptr(), self.st()))
        self.sync()
        n = int(nj.cpu().numpy()[0])
        return dict(topi=topi.cpu().numpy(), topw=topw.cpu().numpy(), cnt=cnt.cpu().numpy(), jbase=jbase.cpu().numpy(), njobs=n,
                    gu=gu.cpu().numpy()[:n], dn=dn.cpu().numpy()[:n])

    def f32_f16(self, x):
        dx = self.up(x.astype(np.float32))
        out = self.zeros(x.shape, self.torch.float16)
        self.ok(self.lib.fnx_f32_f16(dx.data_ptr(), x.size, out.data_ptr(), self.st()))
        self.sync()
        return out.cpu().numpy()

    def swiglu_h16(self, gu, ffs):
        dg = self.up(gu.astype(np.float32))
        out = self.zeros((gu.shape[0], ffs), self.torch.float16)
        self.ok(self.lib.fnx_swiglu_h16(dg.data_ptr(), ffs, gu.shape[0], out.data_ptr(), self.st()))
        self.sync()
        return out.cpu().numpy()

    def moe_mma(self, w, w_stride, nrows, ncols, jobs, x16, out_rows, packed=False, down=False, cap=None, tile16=False, h16=False):
        """jobs: int32 [njobs][130]; the job count is read from device memory, the arrays hold `cap` jobs"""
        t = self.torch
        cap = cap or len(jobs)
        jpad = np.zeros((cap, 130), dtype=np.int32)
        jpad[:len(jobs)] = jobs
        dw_, dj, dx = self.up(w), self.up(jpad), self.up(np.ascontiguousarray(x16, dtype=np.float16))
        if packed:
            self.ok(self.lib.fnx_iq3s_repack(dw_.data_ptr(), dw_.data_ptr(), w.size // 110 * 256, self.st()))
        out = self.zeros((out_rows, nrows), t.float32)
        W = W0 = self.pkg.dw(dw_, ncols, nrows, packed=packed)
        w_stride0 = w_stride
        if tile16:   # re-laid a second time into the prompt path's layout (w_stride then counts that layout's bytes)
            assert packed
            nmat = w.size // (nrows * ncols // 256 * 110)
            d16 = self.zeros(self.lib.fnx_iq3s_tile16_bytes(nrows, ncols, nmat), t.uint8)
            self.ok(self.lib.fnx_iq3s_tile16(dw_.data_ptr(), d16.data_ptr(), nrows, ncols, nmat, self.st()))
            W = self.pkg.dw(d16, ncols, nrows, tile16=True)
            w_stride = self.lib.fnx_iq3s_tile16_bytes(nrows, ncols, 1) if w_stride else 0
        nj = self.up(np.array([len(jobs)], dtype=np.int32))
        if h16:   # nrows = 2 ffs stacked: h = silu(gate) * up as f16 from one launch (tile16), and from the two operators one after the other (unit64)
            ffs = nrows // 2
            one, two = self.zeros((out_rows, ffs), t.float16), self.zeros((out_rows, ffs), t.float16)
            self.ok(self.lib.fnx_moe_gate_up_h16_mma(C.byref(W), w_stride, dj.data_ptr(), nj.data_ptr(), cap, dx.data_ptr(), one.data_ptr(), self.st()))
            self.ok(self.lib.fnx_moe_gate_up_mma(C.byref(W0), w_stride0, dj.data_ptr(), nj.data_ptr(), cap, dx.data_ptr(), out.data_ptr(), self.st()))
            self.ok(self.lib.fnx_swiglu_h16(out.data_ptr(), ffs, out_rows, two.data_ptr(), self.st()))
            self.sync()
            return one.cpu().numpy(), two.cpu().numpy()
        fn = self.lib.fnx_moe_down_mma if down else self.lib.fnx_moe_gate_up_mma
        self.ok(fn(C.byref(W), w_stride, dj.data_ptr(), nj.data_ptr(), cap, dx.data_ptr(), out.data_ptr(), self.st()))
        self.sync()
        return out.cpu().numpy()


    def moe_big(self, w, w_stride, nrows, ncols, jobs, acts, out_rows, down=False, cap=None):
        """the prompt path's jobs over q8_1 activations (fnx_moe_gate_up_big / fnx_moe_down_big), tile16 matrices.
        jobs: int32 [njobs][130]; acts: q8_1 rows as bytes (gate|up), or f32 rows [gate | up] of 2 ncols (down)"""
        t = self.torch
        cap = cap or len(jobs)
        jpad = np.zeros((cap, 130), dtype=np.int32)
        jpad[:len(jobs)] = jobs
        dw_, dj, da = self.up(w), self.up(jpad), self.up(np.ascontiguousarray(acts))
        self.ok(self.lib.fnx_iq3s_repack(dw_.data_ptr(), dw_.data_ptr(), w.size // 110 * 256, self.st()))
        nmat = w.size // (nrows * ncols // 256 * 110)
        d16 = self.zeros(self.lib.fnx_iq3s_tile16_bytes(nrows, ncols, nmat), t.uint8)
        self.ok(self.lib.fnx_iq3s_tile16(dw_.data_ptr(), d16.data_ptr(), nrows, ncols, nmat, self.st()))
        W = self.pkg.dw(d16, ncols, nrows, tile16=True)
        w_stride = self.lib.fnx_iq3s_tile16_bytes(nrows, ncols, 1) if w_stride else 0
        nj = self.up(np.array([len(jobs)], dtype=np.int32))
        out = self.zeros((out_rows, nrows), t.float32)
        fn = self.lib.fnx_moe_down_big if down else self.lib.fnx_moe_gate_up_big
        self.ok(fn(C.byref(W), w_stride, dj.data_ptr(), nj.data_ptr(), cap, da.data_ptr(), out.data_ptr(), self.st()))
        self.sync()
        return out.cpu().numpy()

    # ---- around the MoE half
    def rms_norm_rows(self, x, w, eps):
        dx, dw_ = self.up(x.astype(np.float32)), self.up(w.astype(np.float32))
        y = self.zeros(x.shape, self.torch.float32)
        self.ok(self.lib.fnx_rms_norm_rows(dx.data_ptr(), dw_.data_ptr(), y.data_ptr(), x.shape[0], x.shape[1], eps, self.st()))
        self.sync()
        return y.cpu().numpy()

    def add_norm_q8(self, x, add, w, eps):
        t = self.torch
        rows, n = x.shape
        dx, dw_ = self.up(x.astype(np.float32)), self.up(w.astype(np.float32))
        da = self.up(add.astype(np.float32)) if add is not None else None
        xn, xq = self.zeros((rows, n), t.float32), self.zeros(rows * (n // 32) * 36, t.uint8)
        self.ok(self.lib.fnx_add_norm_q8(dx.data_ptr(), da.data_ptr() if da is not None else None, dw_.data_ptr(), xn.data_ptr(), xq.data_ptr(),
                                         rows, n, eps, self.st()))
        self.sync()
        return dx.cpu().numpy(), xn.cpu().numpy(), xq.cpu().numpy()

    def moe_combine(self, part, topw, sh, sh_logit):
        T, topk = topw.shape
        n = part.shape[1]
        d = [self.up(a.astype(np.float32)) for a in (part, topw, sh, sh_logit)]
        out = self.zeros((T, n), self.torch.float32)
        self.ok(self.lib.fnx_moe_combine(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), 1, out.data_ptr(), T, n, topk, self.st()))
        self.sync()
        return out.cpu().numpy()

    def combine_add_norm_q8(self, part, topw, sh, sh_logit, x, w, eps):
        """part [T * topk][n], topw [T][topk], sh [T][n], sh_logit [T]: returns (x after the add, xn, xq)"""
        t = self.torch
        rows, n = x.shape
        topk = topw.shape[1]
        d = [self.up(a.astype(np.float32)) for a in (part, topw, sh, sh_logit, x, w)]
        xn, xq = self.zeros((rows, n), t.float32), self.zeros(rows * (n // 32) * 36, t.uint8)
        self.ok(self.lib.fnx_combine_add_norm_q8(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), 1, topk, d[4].data_ptr(),
                                                 d[5].data_ptr(), xn.data_ptr(), xq.data_ptr(), rows, n, eps, self.st()))
        self.sync()
        return d[4].cpu().numpy(), xn.cpu().numpy(), xq.cpu().numpy()

    def q8s_tiled(self, dq, rows, cols):
        """the int8 values of a dense matrix (a device tensor [rows][cols]) re-laid tile-major (fnx_q8s_tile): a new tensor"""
        dst = self.zeros(self.lib.fnx_q8s_tile_bytes(rows, cols), self.torch.int8)
        self.ok(self.lib.fnx_q8s_tile(dq.data_ptr(), dst.data_ptr(), rows, cols, self.st()))
        self.sync()
        return dst

    def q8s_gemv(self, q, d, yq, T, tiled=False):
        rows, cols = q.shape
        dq, dd, dy = self.up(q), self.up(d), self.up(yq)
        out = self.zeros((T, rows), self.torch.float32)
        if tiled:
            dq = self.q8s_tiled(dq, rows, cols)
        W = self.pkg.Q8S(dq.data_ptr(), dd.data_ptr(), rows, cols, 1 if tiled else 0)
        self.ok(self.lib.fnx_q8s_gemv(C.byref(W), dy.data_ptr(), out.data_ptr(), rows, T, self.st()))
        self.sync()
        return out.cpu().numpy()

    def attn_prep_append(self, qg, k, v, qn, kn, kc, vc, nq, nkv, pos0, eps, rope):
        t = self.torch
        T = qg.shape[0]
        dq, dk, dv = self.up(qg.astype(np.float32)), self.up(k.astype(np.float32)), self.up(v.astype(np.float32))
        rows = kc.shape[0]
        kc, vc = pad4(kc), pad4(vc)
        dqn, dkn, dkc, dvc = self.up(qn), self.up(kn), self.up(kc), self.up(v_blocked(vc))
        dp = self.up(np.array([pos0], dtype=np.int32))
        r = self.pkg.Rope(*rope)
        self.ok(self.lib.fnx_attn_prep_append(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dqn.data_ptr(), dkn.data_ptr(), dkc.data_ptr(),
                                              dvc.data_ptr(), nq, nkv, T, dp.data_ptr(), kc.shape[0], eps, C.byref(r), self.st()))
        self.sync()
        return dq.cpu().numpy(), dk.cpu().numpy(), dkc.cpu().numpy()[:rows], v_rows(dvc.cpu().numpy())[:rows]

    def attn(self, qg, kc, vc, nq, nkv, pos0):
        t = self.torch
        T = qg.shape[0]
        kc, vc = pad4(kc), pad4(vc)
        max_ctx = kc.shape[0]
        dq, dkc, dvc = self.up(qg.astype(np.float32)), self.up(kc), self.up(v_blocked(vc))
        dp = self.up(np.array([pos0], dtype=np.int32))
        out = self.zeros((T, nq, 256), t.float32)
        scratch = self.zeros(self.lib.fnx_attn_scratch_floats(nq, T, max_ctx), t.float32)
        self.ok(self.lib.fnx_attn(dq.data_ptr(), dkc.data_ptr(), dvc.data_ptr(), out.data_ptr(), nq, nkv, dp.data_ptr(), T, max_ctx,
                                  scratch.data_ptr(), self.st()))
        self.sync()
        return out.cpu().numpy()


def pack_moe_weights(dev, ws, n, ff, packed):
    """ws: the device tensors [gate|up, down, shared gate|up, shared down] as raw ggml blocks. packed: the load-time
    re-laying to unit64, in place (fnx_iq3s_repack). Returns the tensors and their fnx_dw."""
    pkg = dev.pkg
    if packed:
        for w in ws:
            dev.ok(dev.lib.fnx_iq3s_repack(w.data_ptr(), w.data_ptr(), w.numel() // 110 * 256, dev.st()))
    p = bool(packed)
    return ws, [pkg.dw(ws[0], n, 2 * ff, packed=p), pkg.dw(ws[1], ff, n, packed=p), pkg.dw(ws[2], n, 2 * ff, packed=p), pkg.dw(ws[3], ff, n, packed=p)]


class DecoderDev:
    """a SyntheticDecoder on the device: weights, caches, workspace; verify / draft through the C ABI"""

    def __init__(self, dev, model, packed=True, tiled=True):
        """tiled: the dense matrices' int8 values in the tile-major layout (fnx_q8s_tile), as a caller would re-lay them at load"""
        t = dev.torch
        pkg = dev.pkg
        c = model.cfg
        self.dev, self.m, self.c = dev, model, c
        self.keep = []
        n, nq, nkv, ff, nexp, topk = c["n"], c["nq"], c["nkv"], c["ff"], c["nexp"], c["topk"]

        def up(a):
            d = dev.up(a)
            self.keep.append(d)
            return d

        def q8s(tq, rows, cols):
            if tiled:
                dq = dev.q8s_tiled(dev.up(tq[0]), rows, cols)
                self.keep.append(dq)
                return pkg.Q8S(dq.data_ptr(), up(tq[1]).data_ptr(), rows, cols, 1)
            return pkg.Q8S(up(tq[0]).data_ptr(), up(tq[1]).data_ptr(), rows, cols, 0)

        def lay(L):
            ws, dws = pack_moe_weights(dev, [up(L[k]) for k in ("gu", "down", "sh_gu", "sh_down")], n, ff, packed)
            self.keep.extend(ws)
            moe = pkg.MoeLayer(n, ff, nexp, topk, up(L["router"]).data_ptr(), 0, dws[0], 2 * ff * (n // 256) * 110, dws[1], n * (ff // 256) * 110,
                               dws[2], dws[3])
            kc, vc = dev.zeros((c["max_ctx"], nkv, 256), t.float16), dev.zeros((c["max_ctx"], nkv, 256), t.float16)
            self.keep.extend([kc, vc])
            return pkg.DecLayer(up(L["attn_norm"]).data_ptr(), up(L["q_norm"]).data_ptr(), up(L["k_norm"]).data_ptr(), up(L["ffn_norm"]).data_ptr(),
                                q8s(L["wq"], nq * 512, n), q8s(L["wk"], nkv * 256, n), q8s(L["wv"], nkv * 256, n), q8s(L["wo"], n, nq * 256), moe,
                                kc.data_ptr(), vc.data_ptr()), (kc, vc)

        self.layer_arr = (pkg.DecLayer * c["nlayers"])()
        self.caches = []
        for i, L in enumerate(model.layers):
            self.layer_arr[i], kv = lay(L)
            self.caches.append(kv)
        self.D = pkg.Decoder(n, nq, nkv, c["nlayers"], c["vocab"], c["max_ctx"], c["eps"], pkg.Rope(*model.rope),
                             C.cast(self.layer_arr, C.c_void_p), up(model.out_norm).data_ptr(), q8s(model.head, c["vocab"], n),
                             up(model.emb).data_ptr())
        ml, self.mtp_cache = lay(model.mtp["layer"])
        self.M = pkg.Mtp(up(model.mtp["norm_emb"]).data_ptr(), up(model.mtp["norm_hid"]).data_ptr(), up(model.mtp["out_norm"]).data_ptr(),
                         q8s(model.mtp["fc_emb"], n, n), q8s(model.mtp["fc_hid"], n, n), q8s(model.mtp["head"], c["vocab"], n), ml)
        T, P = 16, 16 * topk
        z = dev.zeros
        self.b = dict(x=z((T, n), t.float32), xn=z((T, n), t.float32), qg=z((T, nq * 512), t.float32), k=z((T, nkv * 256), t.float32),
                      v=z((T, nkv * 256), t.float32), att=z((T, nq * 256), t.float32), o=z((T, n), t.float32),
                      attn_scratch=z(dev.lib.fnx_attn_scratch_floats(nq, T, c["max_ctx"]), t.float32), xq=z(T * (max(n, nq * 256) // 32) * 36, t.uint8),
                      hidden=z((T, n), t.float32), logits=z((T, c["vocab"]), t.float32), best_v=z(T, t.float32), best_i=z(T, t.int32),
                      keys=z(pkg.ARGMAX_WORDS, t.int64), err=z(1, t.int32))
        self.mb = dict(xq=z(T * (n // 32) * 36, t.uint8), logits=z((T, nexp + 1), t.float32), topi=z((T, topk), t.int32),
                       topw=z((T, topk), t.float32), jobs_gu=z((P + 1) * 136, t.uint8), jobs_dn=z((P + 1) * 136, t.uint8), njobs=z(2, t.int32), sync=z(pkg.MOE_SYNC_WORDS, t.int32),
                       gu=z((P + T, 2 * ff), t.float32), part=z((P + T, n), t.float32))
        moe_ws = pkg.MoeWs(*(self.mb[k].data_ptr() for k in ("xq", "logits", "topi", "topw", "jobs_gu", "jobs_dn", "njobs", "gu", "part", "sync")))
        self.ws = pkg.DecWs(*[self.b[k].data_ptr() for k in ("x", "xn", "qg", "k", "v", "att", "o", "attn_scratch", "xq", "hidden", "logits",
                                                             "best_v", "best_i", "keys", "err")], moe_ws)
        self.pos = dev.zeros(1, t.int32)

    def caches_numpy(self):
        """every layer's (K, V) as [pos][nkv][256] uint16 arrays, the draft layer's last"""
        out = []
        for kc, vc in self.caches + [self.mtp_cache]:
            k = kc.cpu().numpy().view(np.uint16)
            v = vc.cpu().numpy().view(np.uint16).reshape(self.c["max_ctx"] // V_BLOCK, self.c["nkv"], 256, V_BLOCK)
            out.append((k, v_rows(v)))
        return out

    def set_caches(self, cells):
        """cells: per layer (the draft layer last) a pair of [pos][nkv][256] float16 arrays, written from position 0"""
        for (kc, vc), (k, v) in zip(self.caches + [self.mtp_cache], cells):
            p = k.shape[0]
            assert p % V_BLOCK == 0 and p <= self.c["max_ctx"]
            kc[:p].copy_(self.dev.up(np.ascontiguousarray(k)))
            vc.view(self.dev.torch.float16).reshape(-1)[:v.size].copy_(self.dev.up(v_blocked(v)).reshape(-1))
        self.dev.sync()

    def _result(self, T):
        return dict(hidden=self.b["hidden"].cpu().numpy()[:T], logits=self.b["logits"].cpu().numpy()[:T], best=self.b["best_i"].cpu().numpy()[:T],
                    err=int(self.b["err"].item()))

    def verify(self, tokens, pos0):
        dev = self.dev
        tok = dev.up(np.asarray(tokens, dtype=np.int32))
        self.pos.fill_(pos0)
        dev.ok(dev.lib.fnx_decoder_verify(C.byref(self.D), tok.data_ptr(), len(tokens), self.pos.data_ptr(), C.byref(self.ws), dev.st()))
        dev.sync()
        return self._result(len(tokens))

    def layer(self, x, l, pos0):
        """one layer (l: its number, or -1 for the draft layer's) on the rows x [T][n]: what fnx_decoder_layer leaves in the
        workspace - the rows after the attention half, the attention's rows in q8_1 form (what the output projection read),
        the MoE half's rows - and the router's picks"""
        dev = self.dev
        T = x.shape[0]
        dx = dev.up(np.ascontiguousarray(x, dtype=np.float32))
        self.pos.fill_(pos0)
        L = self.M.layer if l < 0 else self.layer_arr[l]
        dev.ok(dev.lib.fnx_decoder_layer(C.byref(self.D), C.byref(L), dx.data_ptr(), T, self.pos.data_ptr(), C.byref(self.ws), dev.st()))
        dev.sync()
        nb = self.c["nq"] * 256 // 32
        return dict(x_mid=self.b["x"].cpu().numpy()[:T], moe=self.b["o"].cpu().numpy()[:T],
                    att_q8=self.b["xq"].cpu().numpy().reshape(-1)[:T * nb * 36].reshape(T, nb, 36).copy(),
                    topi=self.mb["topi"].cpu().numpy()[:T], err=int(self.b["err"].item()))

    def moe_half(self, x_mid, l, normed=None):
        """the MoE half of layer l (-1: the draft layer's) on the rows x_mid: the norm, then the window. With normed
        rows given the window runs on those instead of the device's own norm of x_mid. Returns (normed rows, output)."""
        dev = self.dev
        T, n = x_mid.shape
        L = self.M.layer if l < 0 else self.layer_arr[l]
        out = dev.zeros((T, n), dev.torch.float32)
        if normed is None:
            dx = dev.up(np.ascontiguousarray(x_mid, dtype=np.float32))
            xn = dev.zeros((T, n), dev.torch.float32)
            dev.ok(dev.lib.fnx_rms_norm_rows(dx.data_ptr(), L.ffn_norm, xn.data_ptr(), T, n, self.c["eps"], dev.st()))
        else:
            xn = dev.up(np.ascontiguousarray(normed, dtype=np.float32))
        dev.ok(dev.lib.fnx_moe_verify_layer(C.byref(L.moe), xn.data_ptr(), T, out.data_ptr(), C.byref(self.ws.moe), dev.st()))
        dev.sync()
        return xn.cpu().numpy(), out.cpu().numpy()

    def routing(self, T):
        """the router logits and picks the last MoE layer run left in the workspace"""
        return self.mb["logits"].cpu().numpy()[:T], self.mb["topi"].cpu().numpy()[:T]

    def verify_routing(self, tokens, pos0):
        """every layer's router logits and picks for this window: the window run at depths 1 .. nlayers (the workspace
        keeps the last layer's; the cells a shallower run writes are the ones the full run writes)"""
        lg, ti = [], []
        for depth in range(1, self.c["nlayers"] + 1):
            self.D.nlayers = depth
            try:
                self.verify(tokens, pos0)
            finally:
                self.D.nlayers = self.c["nlayers"]
            a, b = self.routing(len(tokens))
            lg.append(a)
            ti.append(b)
        return np.stack(lg), np.stack(ti)

    def draft(self, src, tokens, pos0, dv=None, pen=None, par=None):
        """dv = (dv0, dv1): the head's rows for those tokens only; pen = (indexes relative to dv0, counts), par = (repeat, freq,
        present): the last row's penalties"""
        dev = self.dev
        tok = dev.up(np.asarray(tokens, dtype=np.int32))
        dsrc = dev.up(np.ascontiguousarray(src, dtype=np.float32))
        self.pos.fill_(pos0)
        M, keep, T, n = self.M, [], len(tokens), self.c["n"]
        if dv is not None or pen is not None:
            M = type(self.M).from_buffer_copy(self.M)
            if dv is not None:
                M.dv0, M.dv1 = dv
                assert dv[0] % 16 == 0, "a tile-major head is cut at whole tiles of 16 rows"
                M.head = dev.pkg.Q8S(self.M.head.q + dv[0] * n, self.M.head.d + dv[0] * (n // 32) * 2, dv[1] - dv[0], n, self.M.head.tiled)
            if pen is not None:
                keep = [dev.up(np.concatenate([[len(pen[0])], pen[0], pen[1]]).astype(np.int32)), dev.up(np.asarray(par, dtype=np.float32))]
                M.pen, M.pen_par = keep[0].data_ptr(), keep[1].data_ptr()
        dev.ok(dev.lib.fnx_mtp_draft(C.byref(self.D), C.byref(M), dsrc.data_ptr(), tok.data_ptr(), T, self.pos.data_ptr(), C.byref(self.ws), dev.st()))
        dev.sync()
        r = self._result(T)
        if dv is not None:   # the workspace's logits rows are dv1 - dv0 values long in this call
            nv = dv[1] - dv[0]
            r["logits"] = self.b["logits"].cpu().numpy().reshape(-1)[:T * nv].reshape(T, nv)
        return r


class PfLayerDev:
    """One MoE layer's weights plus a chunk workspace, for fnx_moe_prefill_layer."""

    def __init__(self, dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, C_rows, packed=True, tile16=False):
        """tile16 (with packed): the gate|up matrices - and the down matrices, if ff comes in 512s - also in the prompt path's own layout (fnx_iq3s_tile16), which the layer then uses"""
        t = dev.torch
        pkg = dev.pkg
        self.dev, self.n, self.ff, self.nexp, self.topk, self.C = dev, n, ff, nexp, topk, C_rows
        self.router = dev.up(router.astype(np.float32))
        self.gu, self.down, self.sh_gu, self.sh_down = dev.up(gu), dev.up(down), dev.up(sh_gu), dev.up(sh_down)
        self.gu_stride = 2 * ff * (n // 256) * 110
        self.down_stride = n * (ff // 256) * 110
        if packed:
            for w in (self.gu, self.down, self.sh_gu, self.sh_down):
                dev.ok(dev.lib.fnx_iq3s_repack(w.data_ptr(), w.data_ptr(), w.numel() // 110 * 256, dev.st()))
        self.L = pkg.MoeLayer(n, ff, nexp, topk, self.router.data_ptr(), 0, pkg.dw(self.gu, n, 2 * ff, packed=packed), self.gu_stride,
                              pkg.dw(self.down, ff, n, packed=packed), self.down_stride, pkg.dw(self.sh_gu, n, 2 * ff, packed=packed),
                              pkg.dw(self.sh_down, ff, n, packed=packed))
        if tile16:
            assert packed
            lib = dev.lib
            self.gu16 = dev.zeros(lib.fnx_iq3s_tile16_bytes(2 * ff, n, nexp), t.uint8)
            self.sh_gu16 = dev.zeros(lib.fnx_iq3s_tile16_bytes(2 * ff, n, 1), t.uint8)
            dev.ok(lib.fnx_iq3s_tile16(self.gu.data_ptr(), self.gu16.data_ptr(), 2 * ff, n, nexp, dev.st()))
            dev.ok(lib.fnx_iq3s_tile16(self.sh_gu.data_ptr(), self.sh_gu16.data_ptr(), 2 * ff, n, 1, dev.st()))
            self.L.gu = pkg.dw(self.gu16, n, 2 * ff, tile16=True)
            self.L.gu_stride = lib.fnx_iq3s_tile16_bytes(2 * ff, n, 1)
            self.L.sh_gu = pkg.dw(self.sh_gu16, n, 2 * ff, tile16=True)
            if ff % 512 == 0:   # the down matrices too, where their columns come in 512s
                self.down16 = dev.zeros(lib.fnx_iq3s_tile16_bytes(n, ff, nexp), t.uint8)
                self.sh_down16 = dev.zeros(lib.fnx_iq3s_tile16_bytes(n, ff, 1), t.uint8)
                dev.ok(lib.fnx_iq3s_tile16(self.down.data_ptr(), self.down16.data_ptr(), n, ff, nexp, dev.st()))
                dev.ok(lib.fnx_iq3s_tile16(self.sh_down.data_ptr(), self.sh_down16.data_ptr(), n, ff, 1, dev.st()))
                self.L.down = pkg.dw(self.down16, ff, n, tile16=True)
                self.L.down_stride = lib.fnx_iq3s_tile16_bytes(n, ff, 1)
                self.L.sh_down = pkg.dw(self.sh_down16, ff, n, tile16=True)
        P = C_rows * topk
        J, S = P // 64 + nexp, (C_rows + 63) // 64
        self.P, self.J = P, J
        self.bufs = dict(logits=dev.zeros((C_rows, nexp + 1), t.float32), topi=dev.zeros((C_rows, topk), t.int32),
                         topw=dev.zeros((C_rows, topk), t.float32), cnt=dev.zeros(nexp, t.int32), jbase=dev.zeros(nexp, t.int32),
                         jobs_gu=dev.zeros((J + S, 130), t.int32), jobs_dn=dev.zeros((J + S, 130), t.int32), njobs=dev.zeros(2, t.int32),
                         xh=dev.zeros((C_rows, n), t.float16), gu=dev.zeros((P + C_rows, 2 * ff), t.float32),
                         h16=dev.zeros((P + C_rows, ff), t.float16), part=dev.zeros((P + C_rows, n), t.float32))
        self.ws = pkg.PfWs(*[self.bufs[k].data_ptr() for k in ("logits", "topi", "topw", "cnt", "jbase", "jobs_gu", "jobs_dn", "njobs", "xh",
                                                               "gu", "h16", "part")])

    def run(self, x):
        dev = self.dev
        Cn = x.shape[0]
        dx = dev.up(x.astype(np.float32))
        out = dev.zeros((Cn, self.n), dev.torch.float32)
        dev.ok(dev.lib.fnx_moe_prefill_layer(C.byref(self.L), dx.data_ptr(), Cn, out.data_ptr(), C.byref(self.ws), dev.st()))
        dev.sync()
        r = {k: v.cpu().numpy() for k, v in self.bufs.items()}
        r["out"] = out.cpu().numpy()
        return r


class MoeLayerDev:
    """One MoE layer's weights on the device plus a workspace, for fnx_moe_verify_layer and the per-op calls."""

    def __init__(self, dev, n, ff, nexp, topk, router, gu, down, sh_gu, sh_down, T=16, packed=False, sh_q8=None):
        """sh_q8: the shared expert as split Q8_0 instead of IQ3_S blocks: ((q, d) of gate|up, (q, d) of down)"""
        t = dev.torch
        self.dev, self.n, self.ff, self.nexp, self.topk = dev, n, ff, nexp, topk
        pkg = dev.pkg
        self.router = dev.up(router.astype(np.float32))
        self.gu, self.down, self.sh_gu, self.sh_down = dev.up(gu), dev.up(down), dev.up(sh_gu), dev.up(sh_down)
        self.gu_stride = 2 * ff * (n // 256) * 110
        self.down_stride = n * (ff // 256) * 110
        # the load-time re-laying, in place
        (self.gu, self.down, self.sh_gu, self.sh_down), dws = pack_moe_weights(dev, [self.gu, self.down, self.sh_gu, self.sh_down], n, ff, packed)
        self.L = pkg.MoeLayer(n, ff, nexp, topk, self.router.data_ptr(), 0, dws[0], self.gu_stride, dws[1], self.down_stride, dws[2], dws[3])
        if sh_q8 is not None:
            self.q8 = [dev.up(a) for pair in sh_q8 for a in pair]
            self.L.sh_gu_q8 = pkg.Q8S(self.q8[0].data_ptr(), self.q8[1].data_ptr(), 2 * ff, n)
            self.L.sh_down_q8 = pkg.Q8S(self.q8[2].data_ptr(), self.q8[3].data_ptr(), n, ff)
            self.L.sh_gu.p = self.L.sh_down.p = None   # not to be read
        P = T * topk
        self.P = P
        self.xq = dev.zeros(T * (n // 32) * 36, t.uint8)
        self.logits = dev.zeros((T, nexp + 1), t.float32)
        self.topi = dev.zeros((T, topk), t.int32)
        self.topw = dev.zeros((T, topk), t.float32)
        self.jobs_gu = dev.zeros((P + 1) * 136, t.uint8)
        self.jobs_dn = dev.zeros((P + 1) * 136, t.uint8)
        self.njobs = dev.zeros(2, t.int32)
        self.sync = dev.zeros(pkg.MOE_SYNC_WORDS, t.int32)
        self.gu_out = dev.zeros((P + T, 2 * ff), t.float32)
        self.part = dev.zeros((P + T, n), t.float32)
        self.ws = pkg.MoeWs(self.xq.data_ptr(), self.logits.data_ptr(), self.topi.data_ptr(), self.topw.data_ptr(), self.jobs_gu.data_ptr(),
                            self.jobs_dn.data_ptr(), self.njobs.data_ptr(), self.gu_out.data_ptr(), self.part.data_ptr(), self.sync.data_ptr())

    def run(self, x):
        dev = self.dev
        T = x.shape[0]
        dx = dev.up(x.astype(np.float32))
        out = dev.zeros((T, self.n), dev.torch.float32)
        dev.ok(dev.lib.fnx_moe_verify_layer(C.byref(self.L), dx.data_ptr(), T, out.data_ptr(), C.byref(self.ws), dev.st()))
        dev.sync()
        return dict(out=out.cpu().numpy(), logits=self.logits.cpu().numpy()[:T], topi=self.topi.cpu().numpy()[:T],
                    topw=self.topw.cpu().numpy()[:T], njobs=int(self.njobs.cpu().numpy()[0]),
                    gu=self.gu_out.cpu().numpy(), part=self.part.cpu().numpy(),
                    jobs_gu=self.jobs_gu.cpu().numpy().view(JOB_DTYPE), jobs_dn=self.jobs_dn.cpu().numpy().view(JOB_DTYPE),
                    sync=self.sync.cpu().numpy().view(np.uint32))
